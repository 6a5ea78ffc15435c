"""Parity of the HIP path with the CPU oracle, through the C-ABI.

Integer, byte and index results must be bit-exact.  fp32 results are produced
by the same sequence of correctly rounded binary32 operations as the oracle's,
so they are compared bit-exactly too (the stated tolerance, 1e-6 relative /
1 ulp, is therefore met with zero slack).
"""
import json
import os

import numpy as np
import pytest

import oracle_lib
from om_mi355x import workloads as wl

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "onnx_node_vectors.json")) as f:
    GOLD = json.load(f)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def same_f32(a, b):
    """Bit-equal, except that NaN payloads are not compared."""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    return a.shape == b.shape and bool(np.all((bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b))))


# --------------------------------------------------------------------------
# golden vectors through the GPU
# --------------------------------------------------------------------------
def test_device_is_gfx950(rt):
    info = rt.device_info()
    print("device:", info, flush=True)
    assert info["arch"].startswith("gfx950")
    assert rt.init_compatible(rt.VERSION)


def test_golden_vectors_on_gpu(rt):
    g = GOLD["quantizelinear"]
    y = rt.QuantizeLinear(np.array(g["x"], np.float32), np.float32(g["scale"]), np.array(g["zp"], np.uint8))
    assert y.tolist() == g["y"]
    g = GOLD["quantizelinear_axis"]
    y = rt.QuantizeLinear(np.array(g["x"], np.float32).reshape(g["x_shape"]), np.array(g["scale"], np.float32),
                          np.array(g["zp"], np.uint8), axis=1)
    assert y.reshape(-1).tolist() == g["y"]
    g = GOLD["dequantizelinear"]
    y = rt.DequantizeLinear(np.array(g["x"], np.uint8), np.float32(g["scale"]), np.array(g["zp"], np.uint8))
    assert y.tolist() == g["y"]
    g = GOLD["dequantizelinear_axis"]
    y = rt.DequantizeLinear(np.array(g["x"], np.uint8).reshape(g["x_shape"]), np.array(g["scale"], np.float32),
                            np.array(g["zp"], np.uint8), axis=1)
    assert y.reshape(-1).tolist() == g["y"]
    for name in ("dynamicquantizelinear", "dynamicquantizelinear_max_adjusted",
                 "dynamicquantizelinear_min_adjusted"):
        g = GOLD[name]
        y, s, z = rt.DynamicQuantizeLinear(np.array(g["x"], np.float32))
        assert y.tolist() == g["y"] and int(z) == g["zp"] and np.float32(s) == np.float32(g["scale"])
    g = GOLD["matmulinteger"]
    y = rt.MatMulInteger(np.array(g["A"], np.uint8), np.array(g["B"], np.uint8),
                         np.array(g["a_zp"], np.uint8), np.array(g["b_zp"], np.uint8))
    assert y.tolist() == g["Y"]
    for name, dt in (("qlinearmatmul_2D_uint8_float32", np.uint8), ("qlinearmatmul_2D_int8_float32", np.int8)):
        g = GOLD[name]
        for mode in (rt.WRAP, rt.SATURATE):
            y = rt.QLinearMatMul(np.array(g["a"], dt), np.float32(g["a_scale"]), np.array(g["a_zp"], dt),
                                 np.array(g["b"], dt), np.float32(g["b_scale"]), np.array(g["b_zp"], dt),
                                 np.float32(g["y_scale"]), np.array(g["y_zp"], dt), mode)
            assert y.dtype == dt and y.tolist() == g["y"]


# --------------------------------------------------------------------------
# QuantizeLinear / DequantizeLinear
# --------------------------------------------------------------------------
SPECIALS = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 0.0, -0.0, 1e-40, -1e-40,
                     0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.5, 128.5, 254.5, 255.5], np.float32)


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1023, 1024, 4097, 1 << 20, (1 << 20) + 3])
@pytest.mark.parametrize("qdt", [np.uint8, np.int8])
def test_quantize_per_tensor(rt, oracle, n, qdt):
    rng = np.random.default_rng(n)
    x = rng.normal(0, 2, n).astype(np.float32)
    x[: min(n, SPECIALS.size)] = SPECIALS[: min(n, SPECIALS.size)]
    if n > 4000:                       # exact ties: x/s lands on k + 0.5
        x[100:1100] = (np.arange(1000, dtype=np.float32) - 500 + 0.5) * np.float32(0.25)
    for s, zp in [(0.02, 128 if qdt == np.uint8 else -3), (0.25, 0), (1e-38, 7)]:
        zpa = np.array(zp, qdt)
        want = oracle.quantize_linear(x, np.float32(s), zpa)
        got = rt.QuantizeLinear(x, np.float32(s), zpa)
        assert got.dtype == qdt and np.array_equal(got, want), (n, s, zp)
    if qdt == np.uint8:
        assert np.array_equal(rt.QuantizeLinear(x, np.float32(0.02), None),
                              oracle.quantize_linear(x, np.float32(0.02), None))


@pytest.mark.parametrize("qdt", [np.uint8, np.int8])
def test_quantize_every_input_that_does_not_saturate(rt, oracle, qdt):
    """Every binary32 value whose quotient by the scale has a magnitude in
    [1/4, 512), both signs, bit pattern by bit pattern: beyond that range the
    result is the zero point or saturated, which the sampled tests cover.  With
    the scale 1 (the quotient is the input: the rounding alone), a scale whose
    quotients are inexact (reciprocal-multiply path) and a scale small enough
    to take the full divide; about 180 million inputs each."""
    zp = np.array(3 if qdt == np.uint8 else -5, qdt)
    for s in (np.float32(1.0), np.float32(0.0173), np.float32(5e-30)):
        lo = int(np.float32(0.25 * float(s)).view(np.uint32))
        hi = int(np.float32(512.0 * float(s)).view(np.uint32))
        assert hi - lo == 11 << 23
        for start in range(lo, hi, 1 << 24):
            bits = np.arange(start, min(start + (1 << 24), hi), dtype=np.uint32)
            for sign in (0, 0x80000000):
                x = (bits | np.uint32(sign)).view(np.float32)
                got = rt.QuantizeLinear(x, s, zp)
                want = oracle.quantize_linear(x, s, zp, omp=True)
                assert np.array_equal(got, want), (float(s), hex(start), sign)


@pytest.fixture
def quant_mode(rt):
    """Sets the thread's quantization mode for a test and puts 0 back."""
    def set_mode(mode):
        rt.set_quant_mode(mode)
    yield set_mode
    rt.set_quant_mode(0)


@pytest.mark.parametrize("mode", [1, 2, 3])
def test_quantize_dequantize_under_the_compiler_options(rt, oracle, quant_mode, mode):
    """om_mi355x_SetQuantMode: QuantizeLinear with the quotient as x * (1 / scale)
    (--enable-fast-math) and / or without its zero point
    (--disable-quantization-zero-point), DequantizeLinear without its zero
    point, against the oracle's restatement of those lowerings: per-tensor at
    sizes around the kernels' vector width, on a sample where reciprocal and
    divide differ, with special values and scales from tiny to huge; per-axis on
    the last and on an inner axis; misaligned device views."""
    quant_mode(mode)
    assert rt.quant_mode() == mode
    rng = np.random.default_rng(300 + mode)
    sep = np.arange(1, 1601, dtype=np.float32) * np.float32(0.15)   # x / 0.3 against x * (1 / 0.3)
    for qdt in (np.uint8, np.int8):
        zp = np.array(7 if qdt == np.uint8 else -9, qdt)
        for n in (1, 3, 4, 5, 1023, 4097, (1 << 20) + 3):
            x = rng.normal(0, 40, n).astype(np.float32)
            x[: min(n, SPECIALS.size)] = SPECIALS[: min(n, SPECIALS.size)]
            if n > 4000:
                x[100:1700] = sep
            for s in (0.3, 0.0173, 1e-38, 3e38, 2.0 ** -100):
                want = oracle.quantize_linear_mode(x, np.float32(s), zp, mode)
                got = rt.QuantizeLinear(x, np.float32(s), zp)
                assert got.dtype == qdt and np.array_equal(got, want), (qdt, n, s)
        if mode & 1:   # the sample does separate the two forms
            a = oracle.quantize_linear_mode(sep, np.float32(0.3), zp, mode)
            b = oracle.quantize_linear_mode(sep, np.float32(0.3), zp, mode & 2)
            assert (a != b).any()
        # per-axis: last axis and an inner axis
        for shape, axis in (((37, 100), 1), ((5, 6, 70), 1), ((300, 4099), 1)):
            x = rng.normal(0, 30, shape).astype(np.float32)
            sc = rng.uniform(0.05, 2.0, shape[axis]).astype(np.float32)
            z = _rand_q(rng, qdt, (shape[axis],))
            assert np.array_equal(rt.QuantizeLinear(x, sc, z, axis=axis),
                                  oracle.quantize_linear_mode(x, sc, z, mode, axis=axis)), (shape, axis)
            q = _rand_q(rng, qdt, shape)
            want = oracle.dequantize_linear(q, sc, None if mode & 2 else z, axis=axis)
            assert same_f32(rt.DequantizeLinear(q, sc, z, axis=axis), want), (shape, axis)
        q = _rand_q(rng, qdt, (70001,))
        want = oracle.dequantize_linear(q, np.float32(0.02), None if mode & 2 else zp)
        assert same_f32(rt.DequantizeLinear(q, np.float32(0.02), zp), want)
    # a device view 4 bytes off the 16-byte grid (input) and 1 byte off (output)
    n = 5000
    x = rng.normal(0, 40, n + 1).astype(np.float32)
    dx = rt.DeviceArray.from_numpy(x)
    dy = rt.DeviceArray.from_numpy(np.full(n + 8, 0xAB, np.uint8))
    zp = np.array(9, np.uint8)
    rt.QuantizeLinear(rt.DeviceArray.view_of(dx, 1, (n,)), np.float32(0.3), zp, out=rt.DeviceArray.view_of(dy, 1, (n,)))
    rt.synchronize()
    whole = dy.numpy()
    assert whole[0] == 0xAB and (whole[n + 1:] == 0xAB).all()
    assert np.array_equal(whole[1:n + 1], oracle.quantize_linear_mode(x[1:], np.float32(0.3), zp, mode))
    dx.free()
    dy.free()
    with pytest.raises(rt.RuntimeError_, match="SetQuantMode"):
        rt.set_quant_mode(4)
    assert rt.quant_mode() == mode


@pytest.mark.parametrize("mode", [1, 2, 3])
def test_dynamic_quantize_under_the_compiler_options(rt, oracle, quant_mode, mode):
    """DynamicQuantizeLinear and the fused layer under om_mi355x_SetQuantMode:
    zero point 0 and not added without zero points, reciprocal quotient with
    fast math, the scale unchanged; sizes that take the one-block kernel and the
    two-launch path, device-resident operands, and the whole layer
    (DynQuantMatMulDequant) at few rows and at many."""
    quant_mode(mode)
    rng = np.random.default_rng(310 + mode)
    for n, lo, hi in ((1, -1, 1), (100, 0.5, 9), (4096, -3, 5), (16385, -7, -1), (100003, -3, 5), (1 << 20, -2, 6)):
        x = rng.uniform(lo, hi, n).astype(np.float32)
        y, s, z = rt.DynamicQuantizeLinear(x)
        wy, ws, wz = oracle.dynamic_quantize_linear_mode(x, mode)
        assert s == ws and z == wz and np.array_equal(y, wy), (n, lo, hi)
        if mode & 2:
            assert z == 0
    x = rng.uniform(-3, 5, (512, 768)).astype(np.float32)
    dX = rt.DeviceArray.from_numpy(x)
    dy, ds, dz = rt.DynamicQuantizeLinear(dX)
    rt.synchronize()
    wy, ws, wz = oracle.dynamic_quantize_linear_mode(x, mode)
    assert np.array_equal(dy.numpy(), wy) and ds.numpy() == ws and dz.numpy() == wz
    for d in (dX, dy, ds, dz):
        d.free()
    for M, K, N in ((4, 4096, 256), (300, 768, 1000), (512, 768, 3072)):
        x = rng.uniform(-2, 3, (M, K)).astype(np.float32)
        W = _rand_q(rng, np.int8, (K, N))
        ws_ = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        aq, a_s, a_zp = oracle.dynamic_quantize_linear_mode(x, mode)
        want = oracle.dequant_epilogue(oracle.matmul_integer(aq, W, a_zp, None), a_s, ws_)
        assert same_f32(rt.DynQuantMatMulDequant(x, W, None, ws_), want), (M, K, N)


def test_quantize_zero_and_denormal_scale(rt, oracle):
    x = np.array([0.0, -0.0, 1.0, -1.0, np.nan, 3e-45, -3e-45], np.float32)
    for s in (0.0, 1e-45, 1e-39):
        want = oracle.quantize_linear(x, np.float32(s), np.array(9, np.uint8))
        assert np.array_equal(rt.QuantizeLinear(x, np.float32(s), np.array(9, np.uint8)), want), s


def _boundary_points(s):
    """Inputs whose quotient by the scale s lies next to a rounding boundary:
    the floats within three ulps of (k + 1/2) * s and of k * s for |k| <= 300
    (beyond +-256 every 8-bit result saturates), and the special values."""
    k = np.arange(-300, 301, dtype=np.float64)
    with np.errstate(all="ignore"):
        centres = np.concatenate([(k + 0.5) * float(s), k * float(s)]).astype(np.float32)
    centres = centres[np.isfinite(centres)]
    pts = [(centres.view(np.int32) + d).view(np.float32) for d in range(-3, 4)]
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3e38, -3e38, 1e-45, -1e-45, 1e-38, 1.0, -1.0],
                       np.float32)
    return np.concatenate(pts + [special])


# Scales whose quotients take the reciprocal-multiply-and-correct path (2^-96 ..
# 2^96: ordinary ones, powers of two, significands of all ones or all zeros but
# the last bit, both ends of the range) and scales that take the divide.
_TAME_SCALES = [0.1, 1.0, 0.0173, 3.0, 2.0 ** -20, 1.0 - 2.0 ** -24, 2.0 - 2.0 ** -23, 1.0 + 2.0 ** -23,
                0.005, 0.05, 255.0, 2.0 ** -96, 2.0 ** 96, 1.7e-20, 6.1e27]
_OTHER_SCALES = [2.0 ** -97, 1e-38, 1e-39, 1e-45, 1e30, 3e38, 0.0, -0.5, np.inf, np.nan]


def test_quantize_next_to_every_rounding_boundary(rt, oracle):
    """QuantizeLinear divides by the scale either with the full divide or, for
    scales of ordinary magnitude, with a reciprocal multiply and one exact
    correction.  Both must give rne(x / s) as the reference's divf does
    (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:119-144): checked
    where a one-ulp difference in the quotient would show, next to every
    half-integer and integer quotient, through the per-tensor kernels (small and
    4 Mi-element launch shapes), the per-axis kernels (aligned and ragged rows,
    waves of only ordinary scales and waves that mix in others) and
    DynamicQuantizeLinear's quantization."""
    with np.errstate(all="ignore"):
        for s in _TAME_SCALES + _OTHER_SCALES:
            s = np.float32(s)
            x = _boundary_points(s if np.isfinite(s) and s != 0 else np.float32(1))
            for zp in (np.array(0, np.uint8), np.array(77, np.uint8), np.array(255, np.uint8),
                       np.array(-128, np.int8), np.array(5, np.int8), None):
                want = oracle.quantize_linear(x, s, zp)
                got = rt.QuantizeLinear(x, s, zp)
                assert np.array_equal(got, want), (float(s), zp)
        # the launch shape of large tensors (4 Mi elements and more)
        for s in (np.float32(0.0173), np.float32(2.0 ** -97)):
            x = np.tile(_boundary_points(s), 500)
            assert x.size >= 4 << 20
            zp = np.array(131, np.uint8)
            assert np.array_equal(rt.QuantizeLinear(x, s, zp), oracle.quantize_linear(x, s, zp)), float(s)
        # per-axis: a column per scale, its boundary points down the rows
        rng = np.random.default_rng(48)
        tame = np.concatenate([np.array(_TAME_SCALES, np.float32),
                               rng.uniform(0.005, 0.05, 600).astype(np.float32)])
        for scales in (tame, np.concatenate([tame, np.array(_OTHER_SCALES, np.float32)]),
                       np.concatenate([tame, np.array(_OTHER_SCALES, np.float32)])[:-1][::-1].copy()):
            cols = [_boundary_points(s if np.isfinite(s) and s != 0 else np.float32(1)) for s in scales]
            rows = min(c.size for c in cols)
            x = np.stack([c[:rows] for c in cols], axis=1)
            for qdt in (np.uint8, np.int8):
                info = np.iinfo(qdt)
                zp = rng.integers(info.min, info.max + 1, scales.size).astype(qdt)
                assert np.array_equal(rt.QuantizeLinear(x, scales, zp, axis=1),
                                      oracle.quantize_linear(x, scales, zp, axis=1)), (scales.size, qdt)
            # the axis in the middle: one scale per slab
            x3 = np.ascontiguousarray(x.T[:8].reshape(2, 4, -1)[:, :, :rows // 4 * 4])
            sc3 = scales[:4]
            assert np.array_equal(rt.QuantizeLinear(x3, sc3, None, axis=1),
                                  oracle.quantize_linear(x3, sc3, None, axis=1))
        # DynamicQuantizeLinear: the scale follows from the data; boundary points of that scale
        for lo, hi, n in ((-3.1, 4.4, 1 << 12), (-0.02, 11.0, 1 << 16), (0.0, 2.55, 3 << 20), (-1e-30, 1e-30, 5000),
                          (-3e38, 3e38, 70000), (-1e-39, 2e-39, 9000)):
            lo, hi = np.float32(lo), np.float32(hi)
            s = (np.maximum(hi, np.float32(0)) - np.minimum(lo, np.float32(0))) / np.float32(255)
            pts = _boundary_points(s)
            pts = pts[np.isfinite(pts) & (pts >= lo) & (pts <= hi)]
            x = np.resize(np.concatenate([[lo, hi], pts]).astype(np.float32), n)
            wy, ws, wz = oracle.dynamic_quantize_linear(x)
            gy, gs, gz = rt.DynamicQuantizeLinear(x)
            assert np.float32(gs).view(np.uint32) == np.float32(ws).view(np.uint32), (float(lo), float(hi), n)
            assert int(gz) == int(wz) and np.array_equal(gy, wy), (float(lo), float(hi), n)


@pytest.mark.parametrize("shape,axis", [((64, 1000), 1), ((37, 1023), 1), ((5, 7), 1), ((129, 4096), -1),
                                        ((3, 5, 64, 33), 1), ((6, 100), 0), ((2, 3, 4, 5), 2),
                                        ((1, 3, 3, 2), 1), ((300, 2), 1), ((1000, 6), 1), ((257, 4097), 1),
                                        ((3, 1001), -1), ((4099, 3), 1), ((2, 40001), 1),
                                        ((5, 2048), 1), ((3, 32768), 1), ((2, 65536), 1)])
@pytest.mark.parametrize("qdt", [np.uint8, np.int8])
def test_quantize_dequantize_per_axis(rt, oracle, shape, axis, qdt):
    # per-axis: the oracle applies the reference's per-tensor formula per channel
    # (parity unpinned by the reference itself, which asserts on per-axis)
    rng = np.random.default_rng(abs(hash((shape, axis))) % 2**32)
    x = rng.normal(0, 2, shape).astype(np.float32)
    C = shape[axis]
    sc = rng.uniform(0.005, 0.05, C).astype(np.float32)
    info = np.iinfo(qdt)
    zp = rng.integers(info.min, info.max + 1, C).astype(qdt)
    want = oracle.quantize_linear(x, sc, zp, axis=axis)
    got = rt.QuantizeLinear(x, sc, zp, axis=axis)
    assert np.array_equal(got, want)
    got_nozp = rt.QuantizeLinear(x, sc, None, axis=axis)
    assert np.array_equal(got_nozp, oracle.quantize_linear(x, sc, None, axis=axis))
    wd = oracle.dequantize_linear(want, sc, zp, axis=axis)
    gd = rt.DequantizeLinear(want, sc, zp, axis=axis)
    assert same_f32(gd, wd)
    assert same_f32(rt.DequantizeLinear(want, sc, None, axis=axis),
                    oracle.dequantize_linear(want, sc, None, axis=axis))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 7, 1024, 4099, (1 << 20) + 1])
@pytest.mark.parametrize("xdt", [np.uint8, np.int8, np.int32])
def test_dequantize_per_tensor(rt, oracle, n, xdt):
    rng = np.random.default_rng(n + 17)
    info = np.iinfo(xdt)
    x = rng.integers(info.min, info.max, n, dtype=np.int64).astype(xdt)
    zp = np.array(info.max // 2 - 3, xdt)
    s = np.float32(0.0371)
    assert same_f32(rt.DequantizeLinear(x, s, zp), oracle.dequantize_linear(x, s, zp))
    assert same_f32(rt.DequantizeLinear(x, s, None), oracle.dequantize_linear(x, s, None))


def test_dequantize_int32_per_column(rt, oracle):
    rng = np.random.default_rng(23)
    acc = rng.integers(-2**31, 2**31 - 1, (70, 1027), dtype=np.int64).astype(np.int32)
    sc = rng.uniform(1e-5, 1e-3, 1027).astype(np.float32)
    zp = rng.integers(-1000, 1000, 1027).astype(np.int32)
    assert same_f32(rt.DequantizeLinear(acc, sc, zp, axis=1), oracle.dequantize_linear(acc, sc, zp, axis=1))


@pytest.mark.parametrize("rows,cols", [(8, 3968 + 4), (9, 3969), (37, 3970), (40, 3971), (23, 5001), (64, 4100),
                                       (17, 33001), (200, 4111), (11, 51000), (70, 65537), (16, 4095), (33, 8191)])
def test_long_rows_off_the_cache_lines(rt, oracle, rows, cols):
    """Rows of about 4 Ki elements and more whose starts are not 128-byte aligned in
    the float tensor (cols % 32 != 0) take the kernels that re-align every row to
    cache lines and read scale / zero point from a per-block table: every cols % 4,
    row counts that are no multiple of 8, rows that end inside a block's vector and
    inside its table (the wrap to column 0), both element types, with and without
    zero points, and operands that start 4 bytes (scale) / 1 byte (zero point) / 4
    bytes (x) / 16 bytes (y) into their allocations."""
    rng = np.random.default_rng(rows * 100003 + cols)
    for qdt in (np.uint8, np.int8):
        q = rng.integers(0, 256, (rows, cols), dtype=np.uint8).view(qdt)
        sc = rng.uniform(0.005, 0.05, cols).astype(np.float32)
        zp = rng.integers(0, 256, cols, dtype=np.uint8).view(qdt)
        for z in (zp, None):
            assert same_f32(rt.DequantizeLinear(q, sc, z, axis=1), oracle.dequantize_linear(q, sc, z, axis=1))
        # quantize: values on and next to the rounding boundaries of their column's
        # scale, and (second pass) three columns whose scale takes the divide
        x = ((rng.integers(-300, 300, (rows, cols)) + rng.choice(np.array([0.0, 0.5, 0.4999999, 0.5000001]),
                                                                  (rows, cols))) * sc).astype(np.float32)
        for wild in (False, True):
            s2 = sc.copy()
            if wild:
                s2[rng.integers(0, cols, 3)] = np.float32(1e-38)
            for z in (zp, None):
                if z is None and qdt == np.int8:
                    continue
                assert np.array_equal(rt.QuantizeLinear(x, s2, z, axis=1), oracle.quantize_linear(x, s2, z, axis=1))
    want = oracle.dequantize_linear(q, sc, zp, axis=1)
    n = rows * cols
    dq = rt.DeviceArray.from_numpy(np.concatenate([np.zeros(4, qdt), q.reshape(-1)]))
    ds = rt.DeviceArray.from_numpy(np.concatenate([np.zeros(1, np.float32), sc]))
    dz = rt.DeviceArray.from_numpy(np.concatenate([np.zeros(1, qdt), zp]))
    dy = rt.DeviceArray.from_numpy(np.full(n + 8, -7.0, np.float32))
    yv = rt.DeviceArray.view_of(dy, 4, (rows, cols))
    rt.DequantizeLinear(rt.DeviceArray.view_of(dq, 4, (rows, cols)), rt.DeviceArray.view_of(ds, 1, (cols,)),
                        rt.DeviceArray.view_of(dz, 1, (cols,)), axis=1, out=yv)
    assert same_f32(yv.numpy(), want)
    edge = dy.numpy()
    assert (edge[:4] == -7.0).all() and (edge[-4:] == -7.0).all()     # nothing written outside the view
    # quantize with x 16 bytes, y 4 bytes, scale 4 bytes and zero point 1 byte into their allocations
    dx = rt.DeviceArray.from_numpy(np.concatenate([np.zeros(4, np.float32), x.reshape(-1)]))
    dq2 = rt.DeviceArray.from_numpy(np.full(n + 8, 9, qdt))
    qv = rt.DeviceArray.view_of(dq2, 4, (rows, cols))
    rt.QuantizeLinear(rt.DeviceArray.view_of(dx, 4, (rows, cols)), rt.DeviceArray.view_of(ds, 1, (cols,)),
                      rt.DeviceArray.view_of(dz, 1, (cols,)), axis=1, out=qv)
    assert np.array_equal(qv.numpy(), oracle.quantize_linear(x, sc, zp, axis=1))
    edge = dq2.numpy()
    assert (edge[:4] == 9).all() and (edge[-4:] == 9).all()


def test_misaligned_device_views_are_handled(rt, oracle):
    # tensors that start 4 bytes (x) / 1 byte (y) into a GPU allocation: the
    # 16-byte and 4-byte alignment the fast kernels rely on is lost
    rng = np.random.default_rng(31)
    x = rng.normal(0, 2, 5001).astype(np.float32)
    s, zp = np.float32(0.03), np.array(100, np.uint8)
    dx = rt.DeviceArray.from_numpy(x)
    dy = rt.DeviceArray((6000,), np.uint8)
    xv = rt.DeviceArray.view_of(dx, 1, (5000,))
    yv = rt.DeviceArray.view_of(dy, 1, (5000,))
    rt.QuantizeLinear(xv, s, zp, out=yv)
    want = oracle.quantize_linear(x[1:], s, zp)
    assert np.array_equal(yv.numpy(), want)
    dd = rt.DeviceArray((5004,), np.float32)
    dv = rt.DeviceArray.view_of(dd, 1, (5000,))
    rt.DequantizeLinear(yv, s, zp, out=dv)
    assert same_f32(dv.numpy(), oracle.dequantize_linear(want, s, zp))
    gy, gs, gz = rt.DynamicQuantizeLinear(xv)
    wy, ws, wz = oracle.dynamic_quantize_linear(x[1:])
    assert np.array_equal(gy.numpy(), wy) and gs.numpy().reshape(()) == ws
    # matmul with A starting at an odd address and K not a multiple of 16
    A = rng.integers(0, 256, 40 * 50 + 1).astype(np.uint8)
    B = rng.integers(-128, 128, (50, 30)).astype(np.int8)
    dA = rt.DeviceArray.from_numpy(A)
    Av = rt.DeviceArray.view_of(dA, 1, (40, 50))
    got = rt.MatMulInteger(Av, rt.DeviceArray.from_numpy(B), None, None)
    assert np.array_equal(got.numpy(), oracle.matmul_integer(A[1:].reshape(40, 50), B))


# --------------------------------------------------------------------------
# DynamicQuantizeLinear
# --------------------------------------------------------------------------
# (4096, 768) and (2051, 1031) take the one-launch kernel with 8 float4 per thread,
# (4096, 3072) and (3001, 4099) the one with 32; the last three have 1-3 tail elements.
# (16, 4096), (5, 4100), (16388,), (16385,) and (65540,) lie just above the one-block
# kernel's 16 Ki elements and take the two-launch path.
@pytest.mark.parametrize("shape", [(1,), (6,), (3, 4), (1023,), (128, 768), (257, 1031), (4096, 768),
                                   (16, 4096), (5, 4100), (16388,), (16385,), (65540,),
                                   (2051, 1031), (4096, 3072), (3001, 4099)])
def test_dynamic_quantize(rt, oracle, shape):
    rng = np.random.default_rng(int(np.prod(shape)))
    x = rng.normal(0, 1, shape).astype(np.float32)
    wy, ws, wz = oracle.dynamic_quantize_linear(x)
    gy, gs, gz = rt.DynamicQuantizeLinear(x)
    assert np.float32(gs).view(np.uint32) == np.float32(ws).view(np.uint32)
    assert int(gz) == int(wz)
    assert np.array_equal(gy, wy)


def test_dynamic_quantize_edge_inputs(rt, oracle):
    cases = [np.zeros(100, np.float32),                         # scale 0 -> NaN paths -> all 0
             np.full(77, 3.25, np.float32),                     # all positive: min widened to 0
             np.full(77, -3.25, np.float32),                    # all negative: zp 255
             np.array([np.nan, 1.0, -2.0, np.nan, 0.5], np.float32),   # NaN ignored by min/max, NaN -> 0
             np.array([1e-42, -1e-43, 0.0], np.float32),        # denormals kept
             np.array([3e38, -3e38], np.float32)]               # max - min overflows to inf
    for x in cases:
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        gy, gs, gz = rt.DynamicQuantizeLinear(x)
        assert same_f32(np.float32(gs), np.float32(ws)), x[:4]
        assert int(gz) == int(wz) and np.array_equal(gy, wy), x[:4]


def test_dynamic_quantize_mid_size_with_nan_and_inf(rt, oracle):
    # the one-launch kernel: NaN ignored by min / max and quantized to 0, +inf saturates
    rng = np.random.default_rng(5)
    x = rng.normal(0, 3, 2_200_003).astype(np.float32)
    x[rng.integers(0, x.size, 1000)] = np.nan
    for extra in (None, np.inf):
        if extra is not None:
            x[12345] = extra
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        gy, gs, gz = rt.DynamicQuantizeLinear(x)
        assert same_f32(np.float32(gs), np.float32(ws))
        assert int(gz) == int(wz) and np.array_equal(gy, wy)


def test_dynamic_quantize_barrier_timeout_is_reported():
    """The one-launch kernel waits at a grid barrier for a bounded number of polls.
    With the bound forced to zero from the host every block gives up at once (and
    exits normally).  A call on host tensors waits for its kernels anyway: it
    must notice, redo the op with two launches and return correct results.  A
    call on GPU tensors returns without waiting: the give-up is reported at the
    next synchronisation, and the runtime keeps working afterwards."""
    import subprocess, sys, textwrap
    code = textwrap.dedent("""
        import sys, numpy as np
        sys.path.insert(0, %r)
        import om_mi355x as rt
        x = np.random.default_rng(0).normal(0, 1, (4096, 768)).astype(np.float32)
        lo, hi = np.float32(min(x.min(), 0)), np.float32(max(x.max(), 0))
        want_s = (hi - lo) / np.float32(255)
        mode = sys.argv[1]
        zf = np.float32(np.rint(np.clip(np.float32(0) - lo / want_s, 0, 255)))
        want_y = np.clip(np.rint(x / want_s) + zf, 0, 255).astype(np.uint8)
        if mode == "host":
            y, s, z = rt.DynamicQuantizeLinear(x)
            print("FIRST-OK" if np.float32(s) == want_s and np.array_equal(y, want_y) else "FIRST-BAD")
        elif mode == "fused":
            # the fused layer goes through the same wait-and-redo
            b = np.ones((768, 64), np.int8)
            out = rt.DynQuantMatMulDequant(x, b, None, np.float32(1.0))
            ref = (want_y.astype(np.int32) - np.int32(zf)) @ b.astype(np.int32)
            print("FUSED-OK" if np.array_equal(out, ref.astype(np.float32) * (want_s * np.float32(1.0))) else "FUSED-BAD")
        else:
            dx = rt.DeviceArray.from_numpy(x)
            rt.DynamicQuantizeLinear(dx)
            try:
                rt.synchronize()
                print("NO-ERROR")
            except rt.RuntimeError_ as e:
                print("ERROR-OK" if "barrier" in str(e) else "WRONG-ERROR %%s" %% e)
            y, s, z = rt.DynamicQuantizeLinear(dx)
            rt.synchronize()
            print("RECOVERED" if np.float32(s.numpy()) == want_s else "BAD")
    """ % os.path.join(os.path.dirname(HERE), "onnx-mlir_amd"))
    env = dict(os.environ, OM_MI355X_DQL_SPIN_LIMIT="0")
    out = subprocess.run([sys.executable, "-c", code, "host"], env=env, capture_output=True, text=True, timeout=110)
    assert "FIRST-OK" in out.stdout and "two launches" in out.stderr, out.stdout + out.stderr
    out = subprocess.run([sys.executable, "-c", code, "fused"], env=env, capture_output=True, text=True, timeout=110)
    assert "FUSED-OK" in out.stdout and "two launches" in out.stderr, out.stdout + out.stderr
    out = subprocess.run([sys.executable, "-c", code, "device"], env=env, capture_output=True, text=True, timeout=110)
    assert "ERROR-OK" in out.stdout and "RECOVERED" in out.stdout, out.stdout + out.stderr


def test_perf_report_lines_have_the_reference_format(tmp_path):
    """OM_MI355X_PERF_REPORT=1 makes every entry point synchronous and prints a
    before / after pair per call in the format of src/Runtime/OMInstrument.c:164
    ("==PERF-REPORT==, op, node, before|after, since last, since start")."""
    import re, subprocess, sys, textwrap
    report = tmp_path / "perf.txt"
    code = textwrap.dedent("""
        import sys, numpy as np
        sys.path.insert(0, %r)
        import om_mi355x as rt
        x = np.random.default_rng(0).normal(0, 1, (64, 128)).astype(np.float32)
        y, s, z = rt.DynamicQuantizeLinear(x)
        b = np.random.default_rng(1).integers(-127, 128, (128, 96)).astype(np.int8)
        rt.MatMulInteger(y, b, z, None)
    """ % os.path.join(os.path.dirname(HERE), "onnx-mlir_amd"))
    env = dict(os.environ, OM_MI355X_PERF_REPORT="1", ONNX_MLIR_INSTRUMENT_FILE=str(report))
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr
    lines = report.read_text().strip().splitlines()
    pat = re.compile(r"^==PERF-REPORT==, (onnx\.\w+), (\w+), (before|after), (\d+\.\d{6}), (\d+\.\d{6})$")
    got = [pat.match(l).groups() for l in lines]
    assert [(g[0], g[2]) for g in got] == [("onnx.DynamicQuantizeLinear", "before"), ("onnx.DynamicQuantizeLinear", "after"),
                                           ("onnx.MatMulInteger", "before"), ("onnx.MatMulInteger", "after")]
    assert all(float(g[3]) >= 0 for g in got) and float(got[-1][4]) >= float(got[0][4])


def test_dynamic_quantize_invariants_large(rt):
    # properties that hold at any size: zp in range, the extremes map to 0 / 255
    x = wl.normal_f32(2, 0, (2048, 4099), 2.0)
    y, s, z = rt.DynamicQuantizeLinear(x)
    assert 0 <= int(z) <= 255
    assert y[np.unravel_index(np.argmin(x), x.shape)] == 0
    assert y[np.unravel_index(np.argmax(x), x.shape)] == 255
    assert np.float32(s) == (np.float32(x.max()) - np.float32(x.min())) / np.float32(255)


# --------------------------------------------------------------------------
# MatMulInteger
# --------------------------------------------------------------------------
def _rand_q(rng, dt, shape):
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max + 1, shape).astype(dt)


@pytest.mark.parametrize("adt,bdt", [(np.uint8, np.int8), (np.int8, np.uint8), (np.uint8, np.uint8), (np.int8, np.int8)])
def test_matmulinteger_small_exhaustive_shapes(rt, oracle, adt, bdt):
    rng = np.random.default_rng(41)
    for M in (1, 2, 3, 5, 8):
        for K in (1, 2, 7, 16, 33):
            for N in (1, 3, 8):
                A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, bdt, (K, N))
                for az, bz in ((None, None), (_rand_q(rng, adt, ()), _rand_q(rng, bdt, ())),
                               (_rand_q(rng, adt, (M,)), _rand_q(rng, bdt, (N,)))):
                    want = oracle.matmul_integer(A, B, az, bz)
                    got = rt.MatMulInteger(A, B, az, bz)
                    assert np.array_equal(got, want), (M, K, N, adt, bdt)


@pytest.mark.parametrize("M,K,N", [(4, 256, 200), (40, 100, 33), (300, 128, 260), (2048, 1024, 512)])
def test_fused_epilogue_with_bias(rt, oracle, M, K, N):
    """Linear layers carry a bias: MatMulInteger -> Cast -> Mul(a_scale * b_scale) -> Add(bias).
    The product is rounded to f32 first and the bias added to it, as the two
    ONNX ops would; a bias of one element is broadcast; -0.0 results survive a
    missing bias and a +0.0 bias alike as IEEE addition says."""
    rng = np.random.default_rng(M + 3 * N)
    A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
    az = _rand_q(rng, np.uint8, ())
    a_s = np.float32(0.0173)
    bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    bs[::7] *= np.float32(-1.0)          # negative scales: products of accumulator 0 are -0.0
    acc = oracle.matmul_integer(A, B, az, None)
    prod = oracle.dequant_epilogue(acc, a_s, bs)
    for bias in (rng.normal(0, 3, N).astype(np.float32), np.array([1.5], np.float32),
                 np.zeros(N, np.float32)):
        got = rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, bias)
        assert same_f32(got, prod + bias), bias.shape
    assert same_f32(rt.MatMulIntegerDequant(A, B, az, None, a_s, bs), prod)
    # whole layer
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xq, xs, xz = oracle.dynamic_quantize_linear(x)
    want = oracle.dequant_epilogue(oracle.matmul_integer(xq, B, xz, None), xs, bs)
    bias = rng.normal(0, 3, N).astype(np.float32)
    assert same_f32(rt.DynQuantMatMulDequant(x, B, None, bs, bias), want + bias)
    with pytest.raises(rt.RuntimeError_):
        rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, np.zeros(N + 1, np.float32))


def test_few_rows_quantized_inside_the_gemm(rt, oracle):
    """With at most 32 rows and 32 Ki elements (a decode step) the fused layer
    is one launch: the weight-streaming GEMM quantizes the activation rows
    itself.  Same bits as DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul
    (-> Add): scale and zero point over the whole activation, signed and
    unsigned weights, weight zero points, K a multiple of 16 only, constant,
    all-negative and extreme activations."""
    rng = np.random.default_rng(77)
    shapes = [(1, 4096, 1000), (4, 4096, 300), (6, 4096, 64), (3, 16, 33), (32, 768, 96),
              (5, 1008, 257), (1, 64, 7), (17, 1440, 130), (2, 12288, 40), (8, 4096, 64), (32, 1024, 96)]
    for i, (M, K, N) in enumerate(shapes):
        x = rng.normal(0, 1 + i, (M, K)).astype(np.float32)
        if i == 2:
            x[:] = np.float32(2.5)                      # constant: max adjusted to include 0
        if i == 3:
            x = -np.abs(x)                              # all negative: zero point 255
        if i == 4:
            x[3, 5] = np.float32(3e38)
        bdt = np.uint8 if i % 2 else np.int8
        B = _rand_q(rng, bdt, (K, N))
        bz = _rand_q(rng, bdt, (N,)) if i % 3 == 0 else None
        bs = rng.uniform(1e-3, 1e-2, N if i % 4 else 1).astype(np.float32)
        bias = rng.normal(0, 3, N).astype(np.float32) if i % 2 == 0 else None
        xq, xs, xz = oracle.dynamic_quantize_linear(x)
        want = oracle.dequant_epilogue(oracle.matmul_integer(xq, B, xz, bz), xs, bs)
        if bias is not None:
            want = want + bias
        got = rt.DynQuantMatMulDequant(x, B, bz, bs, bias)
        assert same_f32(got, want), (M, K, N)
    # NaN is ignored by min / max and quantizes to 0; an infinite maximum makes
    # the scale infinite (every finite element then quantizes to the zero point)
    for special in (np.nan, np.inf):
        M, K, N = 2, 256, 70
        x = rng.normal(0, 1, (M, K)).astype(np.float32)
        x[1, 17] = special
        B = _rand_q(rng, np.int8, (K, N))
        bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        xq, xs, xz = oracle.dynamic_quantize_linear(x)
        want = oracle.dequant_epilogue(oracle.matmul_integer(xq, B, xz, None), xs, bs)
        got = rt.DynQuantMatMulDequant(x, B, None, bs)
        y, s_, z_ = rt.DynamicQuantizeLinear(x)
        assert np.array_equal(y, xq) and same_f32(np.float32(s_), xs) and z_ == xz, special
        assert same_f32(got, want), special
    # one element more than the kernel takes: the two-launch path, same result
    M, K, N = 3, 8208, 50
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    B = _rand_q(rng, np.int8, (K, N))
    bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    xq, xs, xz = oracle.dynamic_quantize_linear(x)
    want = oracle.dequant_epilogue(oracle.matmul_integer(xq, B, xz, None), xs, bs)
    assert same_f32(rt.DynQuantMatMulDequant(x, B, None, bs), want)


def test_empty_tensors(rt, oracle):
    """A dynamic dimension can be 0 at run time: every op then returns an empty
    result (or, for K = 0, the value of an empty sum) without launching on
    nothing.  DynamicQuantizeLinear of no elements: min = max = 0 after the
    widening to include 0, so scale 0 and zero point 0."""
    rng = np.random.default_rng(5)
    sc, zp = np.float32(0.1), np.array(3, np.uint8)
    for shape in ((0,), (0, 7), (5, 0)):
        x = np.zeros(shape, np.float32)
        assert rt.QuantizeLinear(x, sc, zp).shape == shape
        assert rt.DequantizeLinear(np.zeros(shape, np.uint8), sc, zp).shape == shape
        y, s, z = rt.DynamicQuantizeLinear(x)
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        assert y.shape == shape and same_f32(np.float32(s), np.float32(ws)) and int(z) == int(wz)
    if True:
        C = 5
        scv = rng.uniform(0.01, 0.1, C).astype(np.float32)
        zpv = rng.integers(0, 256, C).astype(np.uint8)
        assert rt.QuantizeLinear(np.zeros((0, C), np.float32), scv, zpv, axis=1).shape == (0, C)
        assert rt.DequantizeLinear(np.zeros((0, C), np.uint8), scv, zpv, axis=1).shape == (0, C)
    for M, K, N in ((0, 16, 8), (4, 16, 0), (4, 0, 8), (0, 0, 0), (40, 0, 300)):
        A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
        az = np.array(9, np.uint8)
        got = rt.MatMulInteger(A, B, az, None)
        assert got.shape == (M, N) and got.dtype == np.int32
        assert np.array_equal(got, oracle.matmul_integer(A, B, az, None)), (M, K, N)
        bs = rng.uniform(0.001, 0.01, N).astype(np.float32)
        gf = rt.MatMulIntegerDequant(A, B, az, None, np.float32(0.02), bs)
        assert gf.shape == (M, N) and not gf.any()
        Bu = _rand_q(rng, np.uint8, (K, N))
        gq = rt.QLinearMatMul(A, np.float32(0.01), az, Bu, np.float32(0.005), np.array(120, np.uint8),
                              np.float32(0.5), np.array(7, np.uint8))
        wq = oracle.qlinear_matmul(A, np.float32(0.01), az, Bu, np.float32(0.005), np.array(120, np.uint8),
                                   np.float32(0.5), np.array(7, np.uint8))
        assert gq.shape == (M, N) and np.array_equal(gq, wq), (M, K, N)
    x = np.zeros((0, 16), np.float32)
    B = _rand_q(rng, np.int8, (16, 8))
    assert rt.DynQuantMatMulDequant(x, B, None, np.float32(0.02)).shape == (0, 8)
    got = rt.DynQuantMatMulDequant(np.zeros((4, 0), np.float32), _rand_q(rng, np.int8, (0, 8)), None,
                                   np.float32(0.02))
    assert got.shape == (4, 8) and not got.any()


@pytest.mark.parametrize("M,K,N", [(128, 768, 768), (130, 200, 260), (257, 1000, 129), (64, 4096, 192),
                                   (1, 4096, 1000), (4, 640, 11008), (16, 333, 77), (500, 48, 500),
                                   (5, 4112, 100), (17, 2064, 70), (40, 11008, 64), (64, 1008, 130)])
def test_matmulinteger_shapes(rt, oracle, M, K, N):
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
    az = _rand_q(rng, np.uint8, ())
    want = oracle.matmul_integer(A, B, az, None)
    assert np.array_equal(rt.MatMulInteger(A, B, az, None), want)
    azr, bzc = _rand_q(rng, np.uint8, (M,)), _rand_q(rng, np.int8, (N,))
    want = oracle.matmul_integer(A, B, azr, bzc)
    assert np.array_equal(rt.MatMulInteger(A, B, azr, bzc), want)


def test_few_rows_of_awkward_length_or_alignment(rt, oracle):
    """Up to 64 rows whose length is no multiple of 16, or that start at an odd
    address: the runtime copies them to aligned rows padded with their zero
    point and uses the weight-streaming kernel over the padded length.  The
    padding stands for real zeros, so every epilogue must give the bits of the
    unpadded product: scalar, per-row and absent zero points, both operand
    types, weight zero points (row sums of A over the padding), the fused
    layer, a GPU view that starts one byte into its allocation."""
    rng = np.random.default_rng(79)
    for M, K, N in ((16, 4100, 11008), (1, 17, 40), (4, 5, 33), (33, 1001, 130), (64, 4099, 96), (7, 15, 64)):
        for adt, bdt in ((np.uint8, np.int8), (np.int8, np.uint8)):
            A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, bdt, (K, N))
            bz = _rand_q(rng, bdt, (N,))
            for az in (_rand_q(rng, adt, ()), _rand_q(rng, adt, (M,)), None):
                want = oracle.matmul_integer(A, B, az, bz)
                assert np.array_equal(rt.MatMulInteger(A, B, az, bz), want), (M, K, N, adt)
                assert "skinny" in rt.last_gemm_kernel(), rt.last_gemm_kernel()
            az = _rand_q(rng, adt, ())
            a_s, bs = np.float32(0.02), rng.uniform(1e-3, 1e-2, N).astype(np.float32)
            bias = rng.normal(0, 2, N).astype(np.float32)
            want = oracle.dequant_epilogue(oracle.matmul_integer(A, B, az, None), a_s, bs) + bias
            assert same_f32(rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, bias), want), (M, K, N)
            bzq, yz = _rand_q(rng, bdt, ()), _rand_q(rng, adt, ())
            for mode in (rt.WRAP, rt.SATURATE):
                wq = oracle.qlinear_matmul(A, np.float32(0.02), az, B, np.float32(0.01), bzq, np.float32(9.0), yz, mode)
                gq = rt.QLinearMatMul(A, np.float32(0.02), az, B, np.float32(0.01), bzq, np.float32(9.0), yz, mode)
                assert np.array_equal(gq, wq), (M, K, N, mode)
        x = rng.normal(0, 1.5, (M, K)).astype(np.float32)
        W, ws = _rand_q(rng, np.int8, (K, N)), rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        wz = _rand_q(rng, np.int8, (N,))
        xq, xs, xz = oracle.dynamic_quantize_linear(x)
        want = oracle.dequant_epilogue(oracle.matmul_integer(xq, W, xz, wz), xs, ws)
        assert same_f32(rt.DynQuantMatMulDequant(x, W, wz, ws), want), (M, K, N)
        assert "skinny" in rt.last_gemm_kernel(), rt.last_gemm_kernel()
    # rows of a good length that start one byte into a GPU allocation
    M, K, N = 8, 4096, 256
    flat = _rand_q(rng, np.uint8, (M * K + 1,))
    B = _rand_q(rng, np.int8, (K, N))
    dflat = rt.DeviceArray.from_numpy(flat)
    Av = rt.DeviceArray.view_of(dflat, 1, (M, K))
    az = _rand_q(rng, np.uint8, ())
    got = rt.MatMulInteger(Av, rt.DeviceArray.from_numpy(B), rt.DeviceArray.from_numpy(az), None)
    assert np.array_equal(got.numpy(), oracle.matmul_integer(flat[1:].reshape(M, K), B, az, None))
    assert "skinny" in rt.last_gemm_kernel()


def test_few_rows_above_the_in_kernel_limit(rt, oracle):
    """Up to 32 rows on both sides of the number of elements that the blocks of
    the weight-streaming GEMM quantize for themselves (above it,
    DynamicQuantizeLinear runs as a kernel of its own in front).  Same bits as
    DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul (-> Add -> Relu) over:
    rows on both sides of the staging limit of four, K a multiple of 16 only,
    grids of two to 344 blocks, weight zero points, NaN and infinities in the
    activation, device-resident operands, and many calls in a row on the same
    buffers without waiting in between."""
    rng = np.random.default_rng(78)
    shapes = [(16, 4096, 11008), (7, 4096, 352), (8, 4096, 64), (32, 4096, 512), (32, 1024, 96), (3, 8208, 96),
              (4, 6160, 130), (25, 1008, 1000), (32, 784, 70), (9, 2736, 33), (31, 4096 + 16, 480), (2, 16384, 64)]
    for i, (M, K, N) in enumerate(shapes):
        x = rng.normal(0, 1 + i, (M, K)).astype(np.float32)
        if i == 2:
            x[1, 7] = np.nan
            x[5, 4000] = np.float32(-3e38)
        if i == 3:
            x = np.abs(x)                               # all positive: zero point 0
        bdt = np.uint8 if i % 2 else np.int8
        B = _rand_q(rng, bdt, (K, N))
        bz = _rand_q(rng, bdt, (N,)) if i % 3 == 0 else None
        bs = rng.uniform(1e-3, 1e-2, N if i % 4 else 1).astype(np.float32)
        bias = rng.normal(0, 3, N).astype(np.float32) if i % 2 == 0 else None
        xq, xs, xz = oracle.dynamic_quantize_linear(x)
        want = oracle.dequant_epilogue(oracle.matmul_integer(xq, B, xz, bz), xs, bs)
        if bias is not None:
            want = want + bias
        got = rt.DynQuantMatMulDequant(x, B, bz, bs, bias)
        assert same_f32(got, want), (M, K, N)
        if i in (0, 5):
            got = rt.DynQuantMatMulDequant(x, B, bz, bs, bias, activation=rt.ACTIVATION_RELU)
            assert same_f32(got, oracle.relu(want)), (M, K, N)
    # GPU-resident operands, constant weights, calls in a row without waiting in between
    M, K, N = 16, 4096, 2048
    W = _rand_q(rng, np.int8, (K, N))
    ws = rng.uniform(1e-3, 5e-3, N).astype(np.float32)
    dW, dS = rt.DeviceArray.from_numpy(W), rt.DeviceArray.from_numpy(ws)
    rt.mark_constant(dW)
    try:
        xs_ = [rng.normal(0, 1 + j, (M, K)).astype(np.float32) for j in range(6)]
        dxs = [rt.DeviceArray.from_numpy(x) for x in xs_]
        outs = [rt.DynQuantMatMulDequant(dx, dW, None, dS) for dx in dxs for _ in range(3)]
        rt.synchronize()
        for j, x in enumerate(xs_):
            xq, xs1, xz = oracle.dynamic_quantize_linear(x)
            want = oracle.dequant_epilogue(oracle.matmul_integer(xq, W, xz, None), xs1, ws)
            for r in range(3):
                assert same_f32(outs[3 * j + r].numpy(), want), (j, r)
    finally:
        rt.unmark_constant(dW)


@pytest.mark.parametrize("adt", [np.int8, np.uint8])
def test_few_rows_through_lds_all_epilogues(rt, oracle, adt):
    """5 to 64 rows with K a multiple of 16: the weight-streaming kernel stages
    the rows of A through LDS.  Several batches of K steps per wave, a last
    batch that is cut short, K not a multiple of 64, row counts on both sides
    of the 32-row tile, all three epilogues."""
    rng = np.random.default_rng(4242 + (adt is np.int8))
    for M, K, N in ((5, 2048 + 16, 96), (31, 4096 + 336, 40), (32, 3072, 64), (33, 2000, 33),
                    (47, 6160, 72), (64, 4096, 31)):
        A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, np.int8, (K, N))
        az, bz = _rand_q(rng, adt, (M,)), _rand_q(rng, np.int8, (N,))
        acc = oracle.matmul_integer(A, B, az, bz)
        assert np.array_equal(rt.MatMulInteger(A, B, az, bz), acc), (M, K, N)
        a_s = np.float32(0.0173)
        bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = rng.normal(0, 2, N).astype(np.float32)
        want = oracle.dequant_epilogue(acc, a_s, bs) + bias
        assert same_f32(rt.MatMulIntegerDequant(A, B, az, bz, a_s, bs, bias), want), (M, K, N)
        ydt = np.uint8 if M % 2 else np.int8
        azq, bzq, yz = _rand_q(rng, adt, ()), _rand_q(rng, np.int8, ()), _rand_q(rng, ydt, ())
        for mode in (rt.WRAP, rt.SATURATE):
            wq = oracle.qlinear_matmul(A, np.float32(0.02), azq, B, np.float32(0.01), bzq,
                                       np.float32(40.0), yz, mode)
            gq = rt.QLinearMatMul(A, np.float32(0.02), azq, B, np.float32(0.01), bzq,
                                  np.float32(40.0), yz, mode)
            assert np.array_equal(gq, wq), (M, K, N, mode)


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4])
def test_every_gemm_kernel_configuration(rt, oracle, cfg, monkeypatch):
    """The kernel choice is a heuristic; force each configuration in turn (0 stages
    tiles through registers, 1 copies them straight into LDS, 2 streams B
    straight into registers, 3 is 1 with 128 x 64 tiles, 4 keeps the weights in
    registers where the shape allows and is 1 elsewhere) on shapes with ragged
    edges, every operand type and all zero-point forms."""
    monkeypatch.setenv("OM_MI355X_GEMM_TILE", str(cfg))
    rng = np.random.default_rng(100 + cfg)
    for (M, K, N), adt, bdt in (((300, 200, 500), np.uint8, np.int8), ((129, 64, 193), np.int8, np.uint8),
                                ((513, 1000, 257), np.uint8, np.uint8), ((256, 192, 384), np.int8, np.int8)):
        A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, bdt, (K, N))
        az, bz = _rand_q(rng, adt, (M,)), _rand_q(rng, bdt, (N,))
        assert np.array_equal(rt.MatMulInteger(A, B, az, bz), oracle.matmul_integer(A, B, az, bz))
        assert np.array_equal(rt.MatMulInteger(A, B, az[:1], None), oracle.matmul_integer(A, B, az[:1], None))
    c = wl.config3(300, 256, 520)
    want = oracle.qlinear_matmul(c["A"], c["a_scale"], c["a_zp"], c["B"], c["b_scale"], c["b_zp"],
                                 c["y_scale"], c["y_zp"], oracle_lib.WRAP)
    assert np.array_equal(rt.QLinearMatMul(c["A"], c["a_scale"], c["a_zp"], c["B"], c["b_scale"], c["b_zp"],
                                           c["y_scale"], c["y_zp"], rt.WRAP), want)
    x = rng.normal(0, 1, (260, 320)).astype(np.float32)
    W = _rand_q(rng, np.int8, (320, 200))
    ws = rng.uniform(1e-3, 1e-2, 200).astype(np.float32)
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(x)
    wantf = oracle.dequant_epilogue(oracle.matmul_integer(aq, W, a_zp, None), a_s, ws)
    assert same_f32(rt.DynQuantMatMulDequant(x, W, None, ws), wantf)


@pytest.mark.parametrize("forced", [True, False])
def test_weights_in_registers_kernel(rt, oracle, forced, monkeypatch):
    """K = 768 with signed weights and no weight zero point runs k_gemm_i8_wreg
    (weights in registers, rows through LDS) when its 128 x 384 blocks fill the
    device, or when forced.  Shapes with ragged edges on both sides (rows and
    column tiles past the matrix, which the kernel computes and must not store),
    uint8 / int8 / already shifted activations, scalar zero points, both
    epilogues it has, bias, and other shapes that must fall through to the other
    kernels (weight zero point, unsigned weights, per-row zero point, K != 768)."""
    if forced:
        monkeypatch.setenv("OM_MI355X_GEMM_TILE", "4")
        shapes = [(128, 384), (1, 32), (129, 416), (300, 800), (1000, 416), (513, 3104)]
    else:
        shapes = [(4096, 2304), (4097, 3104), (3000, 1536)]
    rng = np.random.default_rng(768 + forced)
    K = 768
    for M, N in shapes:
        for adt in (np.uint8, np.int8):
            A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, np.int8, (K, N))
            az = _rand_q(rng, adt, ())
            acc = oracle.matmul_integer(A, B, az, None)
            assert np.array_equal(rt.MatMulInteger(A, B, az, None), acc), (M, N, adt)
            a_s = np.float32(0.0173)
            bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
            want = oracle.dequant_epilogue(acc, a_s, bs)
            assert same_f32(rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, None), want), (M, N, adt)
        bias = rng.normal(0, 2, N).astype(np.float32)
        assert same_f32(rt.MatMulIntegerDequant(A, B, None, None, a_s, bs[:1], bias),
                        oracle.dequant_epilogue(oracle.matmul_integer(A, B, None, None), a_s, bs[:1]) + bias), (M, N)
        # the fused layer hands the kernel activations that are already minus 128
        if M > 64:
            x = rng.normal(0, 1, (M, K)).astype(np.float32)
            aq, xs, xz = oracle.dynamic_quantize_linear(x)
            wantf = oracle.dequant_epilogue(oracle.matmul_integer(aq, B, xz, None), xs, bs) + bias
            assert same_f32(rt.DynQuantMatMulDequant(x, B, None, bs, bias), wantf), (M, N)
    # not this kernel's: the same calls must still be right
    M, N = (300, 800) if forced else (4096, 1536)
    A, Bu = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.uint8, (K, N))
    B = _rand_q(rng, np.int8, (K, N))
    az, azr, bz = _rand_q(rng, np.uint8, ()), _rand_q(rng, np.uint8, (M,)), _rand_q(rng, np.int8, (N,))
    assert np.array_equal(rt.MatMulInteger(A, Bu, az, None), oracle.matmul_integer(A, Bu, az, None))
    assert np.array_equal(rt.MatMulInteger(A, B, az, bz), oracle.matmul_integer(A, B, az, bz))
    assert np.array_equal(rt.MatMulInteger(A, B, azr, None), oracle.matmul_integer(A, B, azr, None))
    A2, B2 = _rand_q(rng, np.uint8, (M, 704)), _rand_q(rng, np.int8, (704, N))
    assert np.array_equal(rt.MatMulInteger(A2, B2, az, None), oracle.matmul_integer(A2, B2, az, None))


@pytest.mark.parametrize("forced", [True, False])
def test_weights_in_registers_kernel_requantizes(rt, oracle, forced, monkeypatch):
    """QLinearMatMul on k_gemm_i8_wreg: K = 768, signed weights whose (required)
    zero point is all zeros -- a host tensor, or GPU memory declared constant,
    which the runtime reads once -- so that B carries no offset; uint8 and int8
    activations and results, wrapping and saturating, shapes with ragged edges
    (N a multiple of 128: whole lines of 8-bit results), per-column b_scale is
    not part of the op.  A zero point that is not zero, or not known to be,
    takes the other kernels and must give the same bits."""
    if forced:
        monkeypatch.setenv("OM_MI355X_GEMM_TILE", "4")
        shapes = [(128, 384), (129, 512), (300, 896), (1000, 384)]
    else:
        shapes = [(4096, 3072), (4097, 2304)]
    rng = np.random.default_rng(76 + forced)
    K = 768
    for M, N in shapes:
        for adt in (np.uint8, np.int8):
            A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, np.int8, (K, N))
            az, yz = _rand_q(rng, adt, ()), _rand_q(rng, adt, ())
            bz0 = np.zeros((), np.int8)
            a_s, b_s, y_s = np.float32(0.0173), np.float32(0.004), np.float32(0.08)
            for mode, omode in ((rt.WRAP, oracle_lib.WRAP), (rt.SATURATE, oracle_lib.SATURATE)):
                want = oracle.qlinear_matmul(A, a_s, az, B, b_s, bz0, y_s, yz, omode)
                got = rt.QLinearMatMul(A, a_s, az, B, b_s, bz0, y_s, yz, mode)
                assert "wreg" in rt.last_gemm_kernel(), (M, N, rt.last_gemm_kernel())
                assert np.array_equal(got, want), (M, N, adt, mode)
                assert (want == np.iinfo(adt).max).any() and (want == np.iinfo(adt).min).any() or mode == rt.WRAP
        # a per-column zero point of zeros is no zero point either
        got = rt.QLinearMatMul(A, a_s, az, B, b_s, np.zeros(N, np.int8), y_s, yz, rt.SATURATE)
        assert "wreg" in rt.last_gemm_kernel()
        assert np.array_equal(got, want)
        # GPU-resident zero point: only a constant one is looked at
        dz = rt.DeviceArray.from_numpy(np.zeros((), np.int8))
        got = rt.QLinearMatMul(A, a_s, az, B, b_s, dz, y_s, yz, rt.SATURATE)
        assert "wreg" not in rt.last_gemm_kernel() and np.array_equal(got, want)
        rt.mark_constant(dz)
        got = rt.QLinearMatMul(A, a_s, az, B, b_s, dz, y_s, yz, rt.SATURATE)
        assert "wreg" in rt.last_gemm_kernel() and np.array_equal(got, want)
        rt.unmark_constant(dz)
        dz.free()
        # a zero point that is not zero
        bz = np.array(-3, np.int8)
        got = rt.QLinearMatMul(A, a_s, az, B, b_s, bz, y_s, yz, rt.SATURATE)
        assert "wreg" not in rt.last_gemm_kernel()
        assert np.array_equal(got, oracle.qlinear_matmul(A, a_s, az, B, b_s, bz, y_s, yz, oracle_lib.SATURATE))


def test_matmul_random_shapes_around_dispatch_boundaries(rt, oracle):
    """Seeded sweep over shapes that sit on both sides of every dispatch
    condition (M 16/17, 32/33, 64/65, 128/129; K a multiple of 64, of 16, of neither;
    N around 32, 64, 128, 256), all operand types and zero-point forms, the
    three epilogues."""
    rng = np.random.default_rng(2024)
    Ms = [1, 2, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 127, 128, 129, 200, 257]
    Ks = [1, 3, 16, 17, 48, 63, 64, 65, 80, 128, 130, 192, 200, 256, 1000]
    Ns = [1, 5, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300]
    for case in range(400):
        M, K, N = (int(rng.choice(v)) for v in (Ms, Ks, Ns))
        adt, bdt = (rng.choice([np.uint8, np.int8]) for _ in range(2))
        A, B = _rand_q(rng, adt, (M, K)), _rand_q(rng, bdt, (K, N))
        az = [None, _rand_q(rng, adt, ()), _rand_q(rng, adt, (M,))][int(rng.integers(0, 3))]
        bz = [None, _rand_q(rng, bdt, ()), _rand_q(rng, bdt, (N,))][int(rng.integers(0, 3))]
        tag = (case, M, K, N, adt.__name__, bdt.__name__, None if az is None else az.shape,
               None if bz is None else bz.shape)
        acc = oracle.matmul_integer(A, B, az, bz)
        kind = case % 3
        if kind == 0:
            assert np.array_equal(rt.MatMulInteger(A, B, az, bz), acc), tag
        elif kind == 1:
            a_s = np.float32(rng.uniform(0.001, 0.1))
            bs = rng.uniform(1e-3, 1e-2, N if case % 2 else 1).astype(np.float32)
            bias = [None, rng.normal(0, 2, N).astype(np.float32)][case % 4 // 2]
            want = oracle.dequant_epilogue(acc, a_s, bs)
            if bias is not None:
                want = want + bias
            assert same_f32(rt.MatMulIntegerDequant(A, B, az, bz, a_s, bs, bias), want), tag
        else:
            ydt = rng.choice([np.uint8, np.int8])
            azq = _rand_q(rng, adt, ()) if az is None else az
            bzq = _rand_q(rng, bdt, ()) if bz is None else bz
            yz = _rand_q(rng, ydt, ())
            a_s, b_s, y_s = (np.float32(v) for v in (0.02, 0.01, rng.uniform(0.05, 2.0)))
            for mode in (rt.WRAP, rt.SATURATE):
                want = oracle.qlinear_matmul(A, a_s, azq, B, b_s, bzq, y_s, yz, mode)
                got = rt.QLinearMatMul(A, a_s, azq, B, b_s, bzq, y_s, yz, mode)
                assert np.array_equal(got, want), tag + (mode,)


def test_quantize_random_shapes_and_axes(rt, oracle):
    """Seeded sweep over ranks 1-4, every axis, per-tensor and per-axis
    parameters, both output types, for QuantizeLinear, DequantizeLinear (8-bit
    and int32 input) and DynamicQuantizeLinear."""
    rng = np.random.default_rng(4048)
    dims = [1, 2, 3, 4, 5, 7, 8, 16, 31, 33, 64, 100, 257]
    for case in range(300):
        rank = int(rng.integers(1, 5))
        shape = tuple(int(rng.choice(dims)) for _ in range(rank))
        axis = int(rng.integers(-rank, rank))
        x = rng.normal(0, 3, shape).astype(np.float32)
        qdt = rng.choice([np.uint8, np.int8])
        info = np.iinfo(qdt)
        C = shape[axis] if case % 3 else 1
        sc = rng.uniform(0.005, 0.5, C).astype(np.float32)
        zp = rng.integers(info.min, info.max + 1, C).astype(qdt) if case % 4 else None
        if C == 1:
            sc = sc.reshape(())
            zp = None if zp is None else zp.reshape(())
        tag = (case, shape, axis, qdt.__name__, C, zp is None)
        wq = oracle.quantize_linear(x, sc, zp, axis=axis, out_dtype=qdt)
        gq = rt.QuantizeLinear(x, sc, zp, axis=axis) if zp is not None or qdt == np.uint8 else None
        if gq is not None:
            assert np.array_equal(gq, wq), tag
        assert same_f32(rt.DequantizeLinear(wq, sc, zp, axis=axis),
                        oracle.dequantize_linear(wq, sc, zp, axis=axis)), tag
        xi = rng.integers(-70000, 70000, shape).astype(np.int32)
        zi = None if zp is None else zp.astype(np.int32)
        assert same_f32(rt.DequantizeLinear(xi, sc, zi, axis=axis),
                        oracle.dequantize_linear(xi, sc, zi, axis=axis)), tag
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        gy, gs, gz = rt.DynamicQuantizeLinear(x)
        assert np.array_equal(gy, wy) and same_f32(np.float32(gs), ws) and int(gz) == int(wz), tag


def test_last_axis_shapes_around_kernel_boundaries(rt, oracle):
    """Per-axis quantize / dequantize on the innermost axis with row lengths on both
    sides of every length the dispatch looks at (2 Ki and 32 Ki powers of two, the
    3968 columns from which rows are re-aligned to cache lines, multiples of 4 and of
    32 and their neighbours, rows that wrap inside a block's table), row counts on
    both sides of 8 and of the rows a block takes, 2-D and 3-D shapes, both element
    types, with and without zero points."""
    rng = np.random.default_rng(777)
    lengths = [2047, 2048, 2049, 2080, 3967, 3968, 3969, 3970, 3971, 3972, 4000, 4095, 4096, 4097, 4100, 4128,
               5119, 5120, 5121, 6000, 8191, 8192, 8193, 16380, 16384, 32764, 32767, 32768, 32769, 33001, 65535, 65537]
    for case, cols in enumerate(lengths):
        rows = int(rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 31]))
        shape = (rows, cols) if case % 3 else (2, max(1, rows // 2), cols)
        qdt = (np.uint8, np.int8)[case % 2]
        x = rng.normal(0, 3, shape).astype(np.float32)
        sc = rng.uniform(0.005, 0.5, cols).astype(np.float32)
        zp = rng.integers(0, 256, cols, dtype=np.uint8).view(qdt) if case % 4 or qdt == np.int8 else None
        tag = (shape, qdt.__name__, zp is None)
        wq = oracle.quantize_linear(x, sc, zp, axis=-1, out_dtype=qdt)
        assert np.array_equal(rt.QuantizeLinear(x, sc, zp, axis=-1), wq), tag
        assert same_f32(rt.DequantizeLinear(wq, sc, zp, axis=-1), oracle.dequantize_linear(wq, sc, zp, axis=-1)), tag
        assert same_f32(rt.DequantizeLinear(wq, sc, None, axis=-1), oracle.dequantize_linear(wq, sc, None, axis=-1)), tag


def test_per_axis_with_inner_slabs(rt, oracle):
    """Per-channel parameters on an axis that is not the innermost one (NCHW
    activations, [C_out, C_in] weights on axis 0): slabs of `inner` elements
    that are whole float4 take the vectorised slab kernels; the shapes cover
    slabs shorter and longer than a block's stride, few and many channels,
    tensors that end inside a block, and the scalar fallback (inner % 4 != 0 or
    inner < 64)."""
    rng = np.random.default_rng(9090)
    cases = [((2, 3, 64), 1), ((5, 7, 8, 8), 1), ((3, 4, 100), 1), ((2, 300, 260), 1), ((1, 5, 4096), 1),
             ((4, 2, 1028), 1), ((64, 1000), 0), ((3, 2, 5, 68), 1), ((2, 33, 7, 12), 1), ((6, 9, 1024), 0),
             ((2, 3, 62), 1), ((2, 3, 60), 1), ((4, 16, 7, 7), 1), ((1, 1024, 1024), 1)]
    for shape, axis in cases:
        C = shape[axis]
        x = rng.normal(0, 3, shape).astype(np.float32)
        for qdt, with_zp in ((np.uint8, True), (np.int8, True), (np.uint8, False)):
            info = np.iinfo(qdt)
            sc = rng.uniform(0.005, 0.5, C).astype(np.float32)
            zp = rng.integers(info.min, info.max + 1, C).astype(qdt) if with_zp else None
            tag = (shape, axis, qdt.__name__, with_zp)
            wq = oracle.quantize_linear(x, sc, zp, axis=axis, out_dtype=qdt)
            assert np.array_equal(rt.QuantizeLinear(x, sc, zp, axis=axis), wq), tag
            assert same_f32(rt.DequantizeLinear(wq, sc, zp, axis=axis),
                            oracle.dequantize_linear(wq, sc, zp, axis=axis)), tag


@pytest.mark.parametrize("mode", [0, 1])
def test_per_axis_with_inner_slabs_that_are_not_whole_vectors(rt, oracle, quant_mode, mode):
    """Per-channel parameters on an inner axis whose slabs are not a whole number
    of float4 (NCHW activations with 7 x 7 or 57 x 57 pixels a channel): walked
    as flat vectors that span two channels at most.  Slabs from four elements
    (the shortest that kernel takes) to thousands, one to many channels per
    block, tensors that end inside a vector, scales that take the divide, the
    three-element slabs that stay with the general kernel, device views off the
    alignment the kernel needs; in the default mode and with the quotient as
    x * (1 / scale)."""
    quant_mode(mode)
    rng = np.random.default_rng(9191 + mode)
    cases = [((64, 33, 7, 7), 1), ((3, 5, 7), 1), ((2, 3, 4099), 1), ((1, 2, 5), 1), ((7, 4, 4), 1), ((2, 1000, 6), 1),
             ((5, 9, 57, 57), 1), ((17, 2, 9), 0), ((3, 300, 13), 1), ((2, 2, 70001), 1), ((4, 6, 3), 1), ((1, 3, 5, 5), 1)]
    for shape, axis in cases:
        C = shape[axis]
        x = rng.normal(0, 30, shape).astype(np.float32)
        x.reshape(-1)[: min(x.size, SPECIALS.size)] = SPECIALS[: min(x.size, SPECIALS.size)]
        for qdt, with_zp in ((np.uint8, True), (np.int8, True), (np.int8, False)):
            sc = rng.uniform(0.05, 2.0, C).astype(np.float32)
            sc[0] = np.float32(1e-38)       # not "tame": the whole wave takes the divide
            zp = _rand_q(rng, qdt, (C,)) if with_zp else None
            tag = (shape, axis, qdt.__name__, with_zp)
            wq = oracle.quantize_linear_mode(x, sc, zp, mode, axis=axis, out_dtype=qdt)
            assert np.array_equal(rt.QuantizeLinear(x, sc, zp, axis=axis) if with_zp else
                                  rt.QuantizeLinear(x, sc, None, axis=axis).view(np.uint8),
                                  wq if with_zp else oracle.quantize_linear_mode(x, sc, None, mode, axis=axis)), tag
            q = _rand_q(rng, qdt, shape)
            assert same_f32(rt.DequantizeLinear(q, sc, zp, axis=axis), oracle.dequantize_linear(q, sc, zp, axis=axis)), tag
    # device views one element off: the kernel's alignment does not hold, results must
    shape = (6, 10, 49)
    n = int(np.prod(shape))
    x = rng.normal(0, 30, n + 1).astype(np.float32)
    sc, zp = rng.uniform(0.05, 2.0, 10).astype(np.float32), _rand_q(rng, np.uint8, (10,))
    dx = rt.DeviceArray.from_numpy(x)
    dq = rt.DeviceArray.from_numpy(np.full(n + 8, 0xAB, np.uint8))
    rt.QuantizeLinear(rt.DeviceArray.view_of(dx, 1, shape), sc, zp, axis=1, out=rt.DeviceArray.view_of(dq, 1, shape))
    rt.synchronize()
    whole = dq.numpy()
    want = oracle.quantize_linear_mode(x[1:].reshape(shape), sc, zp, mode, axis=1)
    assert whole[0] == 0xAB and (whole[n + 1:] == 0xAB).all() and np.array_equal(whole[1:n + 1].reshape(shape), want)
    dy = rt.DeviceArray.from_numpy(np.full(n + 8, -7.0, np.float32))
    rt.DequantizeLinear(rt.DeviceArray.view_of(dq, 1, shape), sc, zp, axis=1, out=rt.DeviceArray.view_of(dy, 1, shape))
    rt.synchronize()
    whole = dy.numpy()
    assert whole[0] == -7.0 and (whole[n + 1:] == -7.0).all()
    assert same_f32(whole[1:n + 1].reshape(shape), oracle.dequantize_linear(want, sc, zp, axis=1))
    for d in (dx, dq, dy):
        d.free()


def test_per_axis_short_rows_of_whole_vectors(rt, oracle):
    """Rows of 4 .. 252 columns (whole float4, fewer than a block of the
    row-walking kernels covers) take the kernels whose threads keep their
    columns from one period of the flat array to the next; 256 columns is the
    first length that stays with the row-walking kernels.  Few rows and many,
    row counts that end inside a period."""
    rng = np.random.default_rng(9292)
    for C in (4, 8, 12, 64, 128, 252, 256):
        for rows in (1, 7, 1000, 65537):
            x = rng.normal(0, 30, (rows, C)).astype(np.float32)
            x.reshape(-1)[: min(x.size, SPECIALS.size)] = SPECIALS[: min(x.size, SPECIALS.size)]
            sc = rng.uniform(0.05, 2.0, C).astype(np.float32)
            for qdt in (np.uint8, np.int8):
                zp = _rand_q(rng, qdt, (C,))
                wq = oracle.quantize_linear(x, sc, zp, axis=1)
                assert np.array_equal(rt.QuantizeLinear(x, sc, zp, axis=1), wq), (C, rows, qdt.__name__)
                assert same_f32(rt.DequantizeLinear(wq, sc, zp, axis=1),
                                oracle.dequantize_linear(wq, sc, zp, axis=1)), (C, rows, qdt.__name__)
            assert np.array_equal(rt.QuantizeLinear(x, sc, None, axis=1), oracle.quantize_linear(x, sc, None, axis=1))


def test_large_gemm_takes_the_wide_tile_path(rt, oracle):
    # big enough for the heuristic to pick the 128 x 256 B-streaming kernel on its own
    rng = np.random.default_rng(77)
    M, K, N = 1024, 2048, 16000
    A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
    az = _rand_q(rng, np.uint8, ())
    assert np.array_equal(rt.MatMulInteger(A, B, az, None), oracle.matmul_integer(A, B, az, None, passes=True))


def test_matmulinteger_extreme_values_wrap(rt, oracle):
    # all-255 x all-(-128) with large K: the int32 accumulator must wrap, not saturate
    M, K, N = 64, 70000, 64
    A = np.full((M, K), 255, np.uint8)
    B = np.full((K, N), -128, np.int8)
    az = np.array(0, np.uint8)
    want = oracle.matmul_integer(A, B, az, None)
    assert want[0, 0] == np.int32((255 * -128 * K + 2**31) % 2**32 - 2**31)
    assert np.array_equal(rt.MatMulInteger(A, B, az, None), want)


def test_matmulinteger_zero_point_identity(rt):
    # Y(A, B, az, bz) == Y(A - az, B - bz, 0, 0) whenever the differences fit in int8
    rng = np.random.default_rng(43)
    A = rng.integers(-50, 50, (100, 300)).astype(np.int8)
    B = rng.integers(-50, 50, (300, 140)).astype(np.int8)
    az, bz = np.array(20, np.int8), rng.integers(-30, 30, 140).astype(np.int8)
    y1 = rt.MatMulInteger(A, B, az, bz)
    y2 = rt.MatMulInteger((A - 20).astype(np.int8), (B - bz[None, :]).astype(np.int8), None, None)
    assert np.array_equal(y1, y2)


def test_matmulinteger_batched_a(rt, oracle):
    rng = np.random.default_rng(44)
    A, B = _rand_q(rng, np.uint8, (3, 5, 64)), _rand_q(rng, np.int8, (64, 24))
    az = _rand_q(rng, np.uint8, ())
    got = rt.MatMulInteger(A, B, az, None)
    assert got.shape == (3, 5, 24) and np.array_equal(got, oracle.matmul_integer(A, B, az, None))


def test_mfma_ceiling_probe(rt):
    """The measurement aid runs, reports a rate between a tenth of and just above
    the published dense int8 peak (5 POP/s) and a plausible shader clock, and
    small-constant operands are not slower than random ones by more than noise."""
    rnd, const = rt.mfma_ceiling(True), rt.mfma_ceiling(False)
    for r in (rnd, const):
        assert 500.0 < r["tops"] < 5300.0 and 0.3 < r["clock_ghz"] < 2.6, r
    assert const["tops"] > 0.9 * rnd["tops"]


def test_fused_relu_epilogue(rt, oracle, monkeypatch):
    """`activation` = Relu on the two fused entry points equals onnx.Relu applied
    to the call's own result without it (max(0, x) is exact), over the kernels a
    shape can take: the weights-in-registers kernel (K = 768), the LDS-staged
    ones, ragged edges, the few-row kernels with and without their own
    quantization, per-row zero points, with and without a bias; a NaN bias
    gives 0, as the reference's maximum does
    (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:746-754)."""
    rng = np.random.default_rng(47)
    for M, K, N in ((512, 768, 3072), (300, 768, 1000), (256, 1024, 512), (130, 200, 70), (4, 4096, 256), (7, 100, 33)):
        A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
        az = _rand_q(rng, np.uint8, ())
        a_s = np.float32(0.013)
        bs = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32) * 3
        bias[N // 2] = np.nan
        for b in (None, bias):
            plain = rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, b)
            got = rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, b, activation=rt.ACTIVATION_RELU)
            want = oracle.relu(plain)
            assert same_f32(got, want), (M, K, N, b is None)
            assert (got >= 0).all() and (got > 0).any() and (got == 0).any()
            # and against the oracle's own chain
            acc = oracle.matmul_integer(A, B, az, None)
            chain = oracle.dequant_epilogue(acc, a_s, bs)
            if b is not None:
                chain = chain + b
            assert same_f32(got, oracle.relu(chain)), (M, K, N)
        x = rng.standard_normal((M, K)).astype(np.float32)
        plain = rt.DynQuantMatMulDequant(x, B, None, bs, bias)
        got = rt.DynQuantMatMulDequant(x, B, None, bs, bias, activation=rt.ACTIVATION_RELU)
        assert same_f32(got, oracle.relu(plain)), (M, K, N)
    # the weights-in-registers kernel by choice (enough rows to fill the device)
    # and by force, on a ragged row count
    for M, force in ((4096, None), (300, "4")):
        A, B = _rand_q(rng, np.uint8, (M, 768)), _rand_q(rng, np.int8, (768, 3072))
        bs = rng.uniform(1e-3, 1e-2, 3072).astype(np.float32)
        if force:
            monkeypatch.setenv("OM_MI355X_GEMM_TILE", force)
        plain = rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.013), bs)
        got = rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.013), bs, activation=rt.ACTIVATION_RELU)
        assert "wreg" in rt.last_gemm_kernel()
        if force:
            monkeypatch.delenv("OM_MI355X_GEMM_TILE")
        assert same_f32(got, oracle.relu(plain)) and (got == 0).any() and (got > 0).any()
    # per-row zero points take the epilogue's other branch
    A, B = _rand_q(rng, np.int8, (70, 96)), _rand_q(rng, np.uint8, (96, 40))
    azm, bzn = _rand_q(rng, np.int8, (70,)), _rand_q(rng, np.uint8, (40,))
    plain = rt.MatMulIntegerDequant(A, B, azm, bzn, np.float32(0.1), np.float32(0.2))
    got = rt.MatMulIntegerDequant(A, B, azm, bzn, np.float32(0.1), np.float32(0.2), activation=1)
    assert same_f32(got, oracle.relu(plain))
    with pytest.raises(rt.RuntimeError_, match="activation"):
        rt.MatMulIntegerDequant(A, B, azm, bzn, np.float32(0.1), np.float32(0.2), activation=3)
    with pytest.raises(rt.RuntimeError_, match="activation"):
        rt.DynQuantMatMulDequant(np.zeros((4, 96), np.float32), B, None, np.float32(0.2), activation=-1)


def test_fused_gelu_epilogue(rt, oracle, monkeypatch):
    """`activation` = Gelu on the two fused entry points against the oracle's
    Gelu of the call's own result without it (that result is bit-exact, see the
    tests above).  PARITY UNPINNED at the bit level: the reference's erf is a
    polynomial approximation its compiler expands, the oracle's is libm's and
    the kernel's an approximation of its own, so the comparison carries a tolerance:
    4 units in the last place of erf (2^-22, erf lies in [-1, 1]) times
    |0.5 x|, the factor the sum 1 + erf is multiplied by, plus one rounding of
    the result.  Shapes as for Relu, so every GEMM kernel is followed by the
    activation once; values from deep in the negative tail (where 1 + erf
    cancels) to large positive ones, NaN and infinities through the bias."""
    rng = np.random.default_rng(53)

    def check(got, plain, what):
        want = oracle.gelu(plain)
        p64 = plain.astype(np.float64)
        tol = np.abs(0.5 * p64) * 2.0 ** -22 + np.abs(want.astype(np.float64)) * 2.0 ** -23 + 1e-45
        fin = np.isfinite(want)
        assert np.array_equal(np.isnan(got), np.isnan(want)), what
        assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)]), what
        err = np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64))
        assert (err <= tol[fin]).all(), (what, float(err.max()))
        # and against the definition in binary64
        from math import erf
        ref = np.array([0.5 * v * (1.0 + erf(v / np.sqrt(2.0))) for v in p64[fin].ravel()[:4096]])
        assert np.allclose(got[fin].ravel()[:4096], ref, rtol=1e-5, atol=1e-6), what

    for M, K, N in ((512, 768, 3072), (300, 768, 1000), (256, 1024, 512), (130, 200, 70), (4, 4096, 256), (7, 100, 33)):
        A, B = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.int8, (K, N))
        az = _rand_q(rng, np.uint8, ())
        # products spread over about [-6, 6]: both tails and the middle of erf
        a_s = np.float32(6.0 / (40.0 * 74.0 * np.sqrt(K)))
        bs = rng.uniform(0.5, 1.0, N).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        bias[N // 2] = np.nan
        bias[N // 3] = np.inf
        bias[N // 4] = -np.inf
        for b in (None, bias):
            plain = rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, b)
            got = rt.MatMulIntegerDequant(A, B, az, None, a_s, bs, b, activation=rt.ACTIVATION_GELU)
            check(got, plain, (M, K, N, b is None))
            assert (plain < -3).any() and (plain > 3).any() and (np.abs(plain) < 0.5).any()
        x = rng.standard_normal((M, K)).astype(np.float32)
        xs = np.float32(6.0 / (0.33 * 74.0 * np.sqrt(K)))
        plain = rt.DynQuantMatMulDequant(x, B, None, bs * xs, bias)
        got = rt.DynQuantMatMulDequant(x, B, None, bs * xs, bias, activation=rt.ACTIVATION_GELU)
        check(got, plain, ("dyn", M, K, N))
    # The weights-in-registers kernel applies Gelu to its results itself, the
    # other kernels leave it to a pass over the output: one function, so the
    # same bits whichever kernel a shape takes.
    A, B = _rand_q(rng, np.uint8, (512, 768)), _rand_q(rng, np.int8, (768, 3072))
    a_s, bs = np.float32(6.0 / (40.0 * 74.0 * np.sqrt(768))), rng.uniform(0.5, 1.0, 3072).astype(np.float32)
    monkeypatch.setenv("OM_MI355X_GEMM_TILE", "4")
    own = rt.MatMulIntegerDequant(A, B, None, None, a_s, bs, activation=2)
    assert "wreg" in rt.last_gemm_kernel()
    x = rng.standard_normal((512, 768)).astype(np.float32)
    xs = bs * np.float32(6.0 / (0.33 * 74.0 * np.sqrt(768)))
    layer = rt.DynQuantMatMulDequant(x, B, None, xs, None, activation=2)
    assert "wreg" in rt.last_gemm_kernel()
    check(layer, rt.DynQuantMatMulDequant(x, B, None, xs, None), "whole layer, weights in registers")
    monkeypatch.setenv("OM_MI355X_GEMM_TILE", "1")
    by_pass = rt.MatMulIntegerDequant(A, B, None, None, a_s, bs, activation=2)
    assert "wreg" not in rt.last_gemm_kernel()
    monkeypatch.delenv("OM_MI355X_GEMM_TILE")
    assert same_f32(own, by_pass)
    # the erf inside, recovered where the division is harmless, against binary64:
    # the bound the header states (2^-22), over the 1.5 million results
    plain = rt.MatMulIntegerDequant(A, B, None, None, a_s, bs).astype(np.float64)
    sel = np.abs(plain) > 0.25
    from scipy.special import erf as erf64
    erf_got = own.astype(np.float64)[sel] / (0.5 * plain[sel]) - 1.0
    m = (plain[sel].astype(np.float32) * np.float32(0.70710678118654752440)).astype(np.float64)
    # (the final product's rounding, half a unit of the result, divided back)
    slack = np.abs(own.astype(np.float64)[sel]) * 2.0 ** -24 / np.abs(0.5 * plain[sel])
    assert (np.abs(erf_got - erf64(m)) <= 2.0 ** -22 + slack).all()
    # an output the caller placed off the 16-byte grid, and batches
    A, B = _rand_q(rng, np.uint8, (3, 37, 64)), _rand_q(rng, np.int8, (64, 23))
    plain = rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.002), np.float32(0.01))
    got = rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.002), np.float32(0.01), activation=2)
    check(got, plain, "batched")
    # results placed 4 and 12 bytes off the 16-byte grid, with guards either side
    A, B = _rand_q(rng, np.uint8, (37, 64)), _rand_q(rng, np.int8, (64, 23))
    plain = rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.002), np.float32(0.01))
    for off in (1, 3):
        buf = rt.DeviceArray.from_numpy(np.full(37 * 23 + 8, -7.0, np.float32))
        rt.MatMulIntegerDequant(A, B, None, None, np.float32(0.002), np.float32(0.01),
                                out=rt.DeviceArray.view_of(buf, off, (37, 23)), activation=2)
        rt.synchronize()
        whole = buf.numpy()
        assert (whole[:off] == -7.0).all() and (whole[off + 37 * 23:] == -7.0).all()
        check(whole[off:off + 37 * 23].reshape(37, 23), plain, ("offset", off))
        buf.free()


def test_matmulinteger_batched_b(rt, oracle):
    """Right-hand sides with batch dimensions (src/Dialect/ONNX/ONNXOps/Math/MatMul.cpp
    :200-292): equal batch dimensions, numpy-style broadcasting on either side, a 2-D
    or 1-D A against a batched B, a 1-D B, and the zero-point forms [.., M, 1] and
    [.., 1, N] that belong to batched operands."""
    rng = np.random.default_rng(45)
    cases = [((2, 3, 5, 64), (2, 3, 64, 24)), ((3, 1, 5, 64), (4, 64, 24)), ((1, 7, 40), (6, 40, 9)),
             ((33, 100), (2, 100, 65)), ((64,), (3, 64, 10)), ((2, 130, 96), (2, 96, 300))]
    for ashape, bshape in cases:
        for adt, bdt in ((np.uint8, np.int8), (np.int8, np.uint8)):
            A, B = _rand_q(rng, adt, ashape), _rand_q(rng, bdt, bshape)
            az, bz = _rand_q(rng, adt, ()), _rand_q(rng, bdt, ())
            want = oracle.matmul_integer(A, B, az, bz)
            got = rt.MatMulInteger(A, B, az, bz)
            assert got.shape == want.shape and np.array_equal(got, want), (ashape, bshape)
            # against numpy's own batched product, in int64
            ref = np.matmul(A.astype(np.int64) - int(az), B.astype(np.int64) - int(bz))
            assert np.array_equal(want.astype(np.int64), ref), (ashape, bshape)
            bzn = _rand_q(rng, bdt, bshape[:-2] + (1, bshape[-1]))
            assert np.array_equal(rt.MatMulInteger(A, B, az, bzn), oracle.matmul_integer(A, B, az, bzn)), (ashape, bshape)
            if len(ashape) >= 2:
                azm = _rand_q(rng, adt, ashape[:-1] + (1,))
                assert np.array_equal(rt.MatMulInteger(A, B, azm, bzn),
                                      oracle.matmul_integer(A, B, azm, bzn)), (ashape, bshape)
    # a 1-D right-hand side (the matrix-vector case of src/Conversion/ONNXToKrnl/Math/MatMul.cpp:299-304)
    A, v = _rand_q(rng, np.uint8, (9, 50)), _rand_q(rng, np.int8, (50,))
    az = _rand_q(rng, np.uint8, ())
    got = rt.MatMulInteger(A, v, az, None)
    assert got.shape == (9,) and np.array_equal(got, oracle.matmul_integer(A, v, az, None))
    assert np.array_equal(got.astype(np.int64), (A.astype(np.int64) - int(az)) @ v.astype(np.int64))
    # device-resident batched operands
    A, B = _rand_q(rng, np.uint8, (4, 70, 128)), _rand_q(rng, np.int8, (4, 128, 96))
    dA, dB = rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B)
    dY = rt.MatMulInteger(dA, dB, None, None)
    rt.synchronize()
    assert np.array_equal(dY.numpy(), oracle.matmul_integer(A, B, None, None))


def test_qlinearmatmul_3d(rt, oracle):
    """QLinearMatMul with batched operands: the shapes of the ONNX node tests
    test_qlinearmatmul_3D_{uint8,int8}_float32 that the reference enables
    (test/backend/inference_backend.py:2549-2554) -- [2,2,4] x [2,4,3] -- built by
    stacking the 2-D node-test matrices, so every batch entry has the published
    2-D answer; and larger seeded shapes against the oracle, both narrowing modes."""
    for name, dt in (("qlinearmatmul_2D_uint8_float32", np.uint8), ("qlinearmatmul_2D_int8_float32", np.int8)):
        g = GOLD[name]
        a, b = np.array(g["a"], dt), np.array(g["b"], dt)
        a3, b3 = np.stack([a, a]), np.stack([b, b])
        y = rt.QLinearMatMul(a3, np.float32(g["a_scale"]), np.array(g["a_zp"], dt), b3,
                             np.float32(g["b_scale"]), np.array(g["b_zp"], dt),
                             np.float32(g["y_scale"]), np.array(g["y_zp"], dt), rt.WRAP)
        assert y.shape == (2, 2, 3)
        assert np.array_equal(y[0], np.array(g["y"], dt)) and np.array_equal(y[1], np.array(g["y"], dt))
    rng = np.random.default_rng(46)
    for dt in (np.uint8, np.int8):
        A, B = _rand_q(rng, dt, (3, 70, 192)), _rand_q(rng, dt, (3, 192, 130))
        az, bz, yz = _rand_q(rng, dt, ()), _rand_q(rng, dt, ()), _rand_q(rng, dt, ())
        for mode in (rt.WRAP, rt.SATURATE):
            want = oracle.qlinear_matmul(A, np.float32(0.02), az, B, np.float32(0.01), bz, np.float32(0.7), yz, mode)
            got = rt.QLinearMatMul(A, np.float32(0.02), az, B, np.float32(0.01), bz, np.float32(0.7), yz, mode)
            assert np.array_equal(got, want), (dt, mode)


def test_constant_weights_are_packed_once_and_stay_correct(rt, oracle):
    rng = np.random.default_rng(45)
    B = _rand_q(rng, np.int8, (256, 384))
    rt.mark_constant(B)
    try:
        for seed in range(3):
            A = _rand_q(np.random.default_rng(seed), np.uint8, (100, 256))
            az = np.array(seed * 40, np.uint8)
            assert np.array_equal(rt.MatMulInteger(A, B, az, None), oracle.matmul_integer(A, B, az, None))
    finally:
        rt.clear_cache()


def test_constant_weight_shared_by_every_kernel_family(rt, oracle):
    """One constant weight, packed once, used in turn with row counts that select
    the skinny kernel, the kernel that copies tiles into LDS and the kernel
    that streams B into registers."""
    rng = np.random.default_rng(46)
    K, N = 128, 16384
    B = _rand_q(rng, np.int8, (K, N))
    bz = _rand_q(rng, np.int8, (N,))
    rt.mark_constant(B)
    try:
        for M in (8, 1024, 130, 1024, 8):
            A = _rand_q(np.random.default_rng(M), np.uint8, (M, K))
            az = np.array(77, np.uint8)
            assert np.array_equal(rt.MatMulInteger(A, B, az, bz), oracle.matmul_integer(A, B, az, bz)), M
    finally:
        rt.clear_cache()


def test_host_buffers_kept_on_device_between_ops(rt, oracle):
    """The compiled-model flow: intermediates are plain host allocations that the
    accelerator pass declares device-backed.  The chain DynamicQuantizeLinear ->
    MatMulInteger -> QuantizeLinear then runs without touching them (they keep
    their sentinel bytes), and the final host output is exact."""
    rng = np.random.default_rng(61)
    M, K, N = 300, 256, 384
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = _rand_q(rng, np.int8, (K, N))
    aq = np.full((M, K), 0xAB, np.uint8)
    a_s = np.full((), -777.0, np.float32)
    a_z = np.full((), 0xCD, np.uint8)
    acc = np.full((M, N), 0x5A5A5A5A, np.int32)
    for t in (aq, a_s, a_z, acc):
        rt.keep_on_device(t)
    try:
        calls = [rt.PreparedCall("om_mi355x_DynamicQuantizeLinear", aq, a_s, a_z, x),
                 rt.PreparedCall("om_mi355x_MatMulInteger", acc, aq, W, a_z, None)]
        for c in calls:
            c()
            c.check()
        got = rt.DequantizeLinear(acc, np.float32(0.5), None)     # host output: staged and copied back
        waq, ws, wz = oracle.dynamic_quantize_linear(x)
        want = oracle.matmul_integer(waq, W, wz, None).astype(np.float32) * np.float32(0.5)
        assert np.array_equal(got, want)
        assert (aq == 0xAB).all() and a_s == np.float32(-777.0) and a_z == 0xCD and (acc == 0x5A5A5A5A).all()
        for c in calls:
            c.close()
    finally:
        for t in (aq, a_s, a_z, acc):
            rt.release(t)
    # after the release the same buffers are ordinary host tensors again
    y, s, z = rt.DynamicQuantizeLinear(x)
    assert np.array_equal(y, waq)
    # a second inference reuses the released GPU blocks; this time another
    # host thread releases, which has to wait for the work queued here
    import threading
    for t in (aq, acc):
        rt.keep_on_device(t)
    rt.QuantizeLinear(x, s, z, out=aq)
    rt.MatMulInteger(aq, W, z, None, out=acc)
    got = rt.DequantizeLinear(acc, np.float32(0.25), None)
    assert np.array_equal(got, oracle.matmul_integer(waq, W, wz, None).astype(np.float32) * np.float32(0.25))
    assert (aq == 0xAB).all() and (acc == 0x5A5A5A5A).all()
    th = threading.Thread(target=lambda: [rt.release(t) for t in (aq, acc)])
    th.start()
    th.join()
    rt.MatMulInteger(waq, W, wz, None, out=acc)
    assert np.array_equal(acc, oracle.matmul_integer(waq, W, wz, None))


def test_large_host_buffers_both_ways(rt, oracle):
    """Large host tensors (inputs from 8 MiB, outputs from 4 MiB) cross PCIe in pieces through page-locked
    slots, shared out between the calling thread and helper threads: sizes that
    are no multiple of a piece, both piece sizes, one piece more than there are
    lanes, and two host threads at once (one of them finds the helpers taken)."""
    import threading
    rng = np.random.default_rng(2024)
    sc, zp = np.float32(0.037), np.array(9, np.uint8)
    sizes = [(1 << 20) + 1, (2 << 20) + 1, (2 << 20) * 3 + 17, 8 * (1 << 20) + 5, 9_000_001, 17_000_003]
    for n in sizes:                       # x: 4n bytes in, y: n bytes out, then the reverse
        x = rng.normal(0, 3, n).astype(np.float32)
        q = rt.QuantizeLinear(x, sc, zp)
        assert np.array_equal(q, oracle.quantize_linear(x, sc, zp)), n
        y = rt.DequantizeLinear(q, sc, zp)        # n bytes in, 4n bytes out
        assert np.array_equal(y, oracle.dequantize_linear(q, sc, zp)), n
    xs = [rng.normal(0, 2, 5_000_003 + 999 * t).astype(np.float32) for t in range(3)]
    want = [oracle.quantize_linear(x, sc, zp) for x in xs]
    errors = []

    def work(t):
        try:
            for _ in range(3):
                q = rt.QuantizeLinear(xs[t], sc, zp)
                assert np.array_equal(q, want[t])
                y = rt.DequantizeLinear(q, sc, zp)
                assert np.array_equal(y, oracle.dequantize_linear(want[t], sc, zp))
        except Exception as e:          # noqa: BLE001
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_concurrent_host_threads(rt, oracle):
    """Entry points are re-entrant: four host threads (each gets its own stream)
    run DynamicQuantizeLinear on a tensor that takes the one-launch kernel,
    MatMulInteger on a shared constant weight and QuantizeLinear at the same time."""
    import threading
    rng = np.random.default_rng(99)
    B = _rand_q(rng, np.int8, (256, 1024))
    rt.mark_constant(B)
    xs = [rng.normal(0, 1 + t, (2100, 1001)).astype(np.float32) for t in range(4)]
    As = [_rand_q(rng, np.uint8, (300 + 64 * t, 256)) for t in range(4)]
    want_dql = [oracle.dynamic_quantize_linear(x) for x in xs]
    want_mm = [oracle.matmul_integer(A, B, np.array(3, np.uint8), None) for A in As]
    sc, zp = np.float32(0.05), np.array(7, np.uint8)
    want_q = [oracle.quantize_linear(x, sc, zp) for x in xs]
    errors = []

    def work(t):
        try:
            for _ in range(3):
                y, s, z = rt.DynamicQuantizeLinear(xs[t])
                assert np.array_equal(y, want_dql[t][0]) and int(z) == int(want_dql[t][2])
                assert np.array_equal(rt.MatMulInteger(As[t], B, np.array(3, np.uint8), None), want_mm[t])
                assert np.array_equal(rt.QuantizeLinear(xs[t], sc, zp), want_q[t])
        except BaseException as e:  # noqa: BLE001 - reported below
            errors.append((t, repr(e)))

    try:
        threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
        for th in threads:
            th.start()
        for th in threads:
            th.join(100)
        assert not errors, errors
        assert not any(th.is_alive() for th in threads)
    finally:
        rt.clear_cache()


# --------------------------------------------------------------------------
# QLinearMatMul and the fused layers at the benchmark configurations
# --------------------------------------------------------------------------
@pytest.mark.parametrize("mode", ["wrap", "saturate"])
def test_config3_qlinearmatmul(rt, oracle, mode):
    c = wl.config3()
    m_rt, m_or = (rt.WRAP, oracle_lib.WRAP) if mode == "wrap" else (rt.SATURATE, oracle_lib.SATURATE)
    want = oracle.qlinear_matmul(c["A"], c["a_scale"], c["a_zp"], c["B"], c["b_scale"], c["b_zp"],
                                 c["y_scale"], c["y_zp"], m_or)
    got = rt.QLinearMatMul(c["A"], c["a_scale"], c["a_zp"], c["B"], c["b_scale"], c["b_zp"],
                           c["y_scale"], c["y_zp"], m_rt)
    assert got.dtype == np.uint8 and np.array_equal(got, want)


def test_qlinearmatmul_int8_and_per_row_column_zero_points(rt, oracle):
    rng = np.random.default_rng(51)
    a, b = _rand_q(rng, np.int8, (70, 130)), _rand_q(rng, np.int8, (130, 90))
    az, bz = _rand_q(rng, np.int8, (70,)), _rand_q(rng, np.int8, (90,))
    for mode_rt, mode_or in ((rt.WRAP, oracle_lib.WRAP), (rt.SATURATE, oracle_lib.SATURATE)):
        want = oracle.qlinear_matmul(a, 0.02, az, b, 0.01, bz, 0.3, np.array(-7, np.int8), mode_or)
        got = rt.QLinearMatMul(a, np.float32(0.02), az, b, np.float32(0.01), bz, np.float32(0.3),
                               np.array(-7, np.int8), mode_rt)
        assert got.dtype == np.int8 and np.array_equal(got, want)


def test_qlinearmatmul_per_column_b_scale(rt, oracle):
    """Per-channel weight scales in QLinearMatMul have no counterpart in the
    reference (its tests and lowering use scalar scales), so this is parity
    unpinned: the expected value composes the oracle's integer matmul with the
    reference's requantize op order, s_j = (a_scale * b_scale[j]) / y_scale."""
    rng = np.random.default_rng(52)
    M, K, N = 200, 192, 384
    a, b = _rand_q(rng, np.uint8, (M, K)), _rand_q(rng, np.uint8, (K, N))
    az, bz = np.array(121, np.uint8), _rand_q(rng, np.uint8, (N,))
    a_s, y_s, yz = np.float32(0.013), np.float32(0.41), np.array(17, np.uint8)
    b_s = rng.uniform(1e-3, 2e-2, N).astype(np.float32)
    acc = oracle.matmul_integer(a, b, az, bz).astype(np.int32)
    sj = ((a_s * b_s).astype(np.float32) / y_s).astype(np.float32)
    q = np.rint(acc.astype(np.float32) * sj[None, :]).astype(np.int64) + int(yz)
    for mode, want in ((rt.WRAP, (q & 0xFF).astype(np.uint8)), (rt.SATURATE, np.clip(q, 0, 255).astype(np.uint8))):
        got = rt.QLinearMatMul(a, a_s, az, b, b_s, bz, y_s, yz, mode)
        assert got.dtype == np.uint8 and np.array_equal(got, want)


def test_config1_graph_separate_ops_and_fused(rt, oracle):
    c = wl.config1()
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(c["A"])
    acc = oracle.matmul_integer(aq, c["B"], a_zp, c["b_zp"])
    want = oracle.dequant_epilogue(acc, a_s, c["b_scale"])
    # the graph as the reference compiles it: three ops, host tensors between them
    gq, gs, gz = rt.DynamicQuantizeLinear(c["A"])
    assert np.array_equal(gq, aq) and np.float32(gs) == a_s and int(gz) == int(a_zp)
    gacc = rt.MatMulInteger(gq, c["B"], gz, c["b_zp"])
    assert np.array_equal(gacc, acc)
    assert same_f32(rt.MatMulIntegerDequant(gq, c["B"], gz, c["b_zp"], gs, c["b_scale"]), want)
    # the fused layer
    assert same_f32(rt.DynQuantMatMulDequant(c["A"], c["B"], c["b_zp"], c["b_scale"]), want)
    assert same_f32(rt.DynQuantMatMulDequant(c["A"], c["B"], None, c["b_scale"]), want)


@pytest.mark.parametrize("name", list(wl.CONFIG4_SHAPES))
def test_config4_layers_reduced_m(rt, oracle, name):
    c = wl.config4(name, M=384)
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(c["X"])
    acc = oracle.matmul_integer(aq, c["W"], a_zp, None)
    want = oracle.dequant_epilogue(acc, a_s, c["w_scale"])
    assert same_f32(rt.DynQuantMatMulDequant(c["X"], c["W"], None, c["w_scale"]), want)


def _check_full_size_layer(rt, oracle, c, sample_rows):
    """A layer at its benchmark size, every element: the int32 accumulator
    against the oracle's OpenMP restatement of the reference's passes (pinned to
    the plain triple loop in tests/test_oracle.py), the fused result against
    that accumulator scaled by the oracle.  Kept from when the oracle was the
    triple loop only: sampled rows (first, last, both sides of tile edges,
    random ones) against that loop, and two checksums over the accumulator
    computed another way -- its column sums must equal (sum of the rows of
    A - zp) x W and its row sums (A - zp) x (sum of the columns of W), in
    arithmetic modulo 2^32."""
    X, W, ws = c["X"], c["W"], c["w_scale"]
    M, K = X.shape
    N = W.shape[1]
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(X)
    got = rt.DynQuantMatMulDequant(X, W, None, ws)
    rng = np.random.default_rng(M + N)
    rows = sorted(set([0, 1, 31, 32, 127, 128, 255, 256, M - 129, M - 128, M - 2, M - 1]
                      + list(rng.integers(0, M, sample_rows))))
    rows = [r for r in rows if 0 <= r < M]
    want = oracle.dequant_epilogue(oracle.matmul_integer(aq[rows], W, a_zp, None), a_s, ws)
    assert same_f32(got[rows], want)
    acc = rt.MatMulInteger(aq, W, a_zp, None)
    # all partial sums stay below 2^53: float64 arithmetic is exact here
    a_colsum = aq.sum(axis=0, dtype=np.int64) - M * int(a_zp)          # [K]
    w_rowsum = W.sum(axis=1, dtype=np.int64)                           # [K]
    want_cols = np.zeros(N, np.float64)
    for k0 in range(0, K, 1024):
        want_cols += a_colsum[k0:k0 + 1024].astype(np.float64) @ W[k0:k0 + 1024].astype(np.float64)
    want_rows = (aq.astype(np.float64) - float(a_zp)) @ w_rowsum.astype(np.float64)
    mod = 1 << 32
    assert np.array_equal(acc.sum(axis=0, dtype=np.int64) % mod, want_cols.astype(np.int64) % mod)
    assert np.array_equal(acc.sum(axis=1, dtype=np.int64) % mod, want_rows.astype(np.int64) % mod)
    # every element of the accumulator, and the fused result is it, scaled
    assert np.array_equal(acc, oracle.matmul_integer(aq, W, a_zp, None, passes=True))
    assert same_f32(got, oracle.dequant_epilogue(acc, a_s, ws))


@pytest.mark.parametrize("name", list(wl.CONFIG4_SHAPES))
def test_config4_layers_full_size(rt, oracle, name):
    _check_full_size_layer(rt, oracle, wl.config4(name), 48)


@pytest.mark.parametrize("name", list(wl.CONFIG5_SHAPES))
def test_config5_prefill_full_size(rt, oracle, name):
    _check_full_size_layer(rt, oracle, wl.config5(name), 12)


@pytest.mark.parametrize("M", [1, 4, 16])
def test_config5_decode_shapes(rt, oracle, M):
    c = wl.config5("up", M=M)
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(c["X"])
    acc = oracle.matmul_integer(aq, c["W"], a_zp, None)
    want = oracle.dequant_epilogue(acc, a_s, c["w_scale"])
    assert same_f32(rt.DynQuantMatMulDequant(c["X"], c["W"], None, c["w_scale"]), want)


def test_fused_layer_with_unsigned_weights_and_zero_points(rt, oracle):
    rng = np.random.default_rng(61)
    x = rng.normal(0, 1, (200, 320)).astype(np.float32)
    W = _rand_q(rng, np.uint8, (320, 150))
    wz = _rand_q(rng, np.uint8, (150,))
    ws = rng.uniform(1e-3, 1e-2, 150).astype(np.float32)
    aq, a_s, a_zp = oracle.dynamic_quantize_linear(x)
    want = oracle.dequant_epilogue(oracle.matmul_integer(aq, W, a_zp, wz), a_s, ws)
    assert same_f32(rt.DynQuantMatMulDequant(x, W, wz, ws), want)


# --------------------------------------------------------------------------
# device-resident operands: used in place, results stay on the GPU
# --------------------------------------------------------------------------
def test_device_resident_chain(rt, oracle):
    c = wl.config4("out", M=512)
    dX = rt.DeviceArray.from_numpy(c["X"])
    dW = rt.DeviceArray.from_numpy(c["W"])
    dS = rt.DeviceArray.from_numpy(c["w_scale"])
    rt.mark_constant(dW)
    try:
        dq, ds, dz = rt.DynamicQuantizeLinear(dX)
        assert isinstance(dq, rt.DeviceArray)
        dacc = rt.MatMulInteger(dq, dW, dz, None)
        dout = rt.MatMulIntegerDequant(dq, dW, dz, None, ds, dS)
        dfused = rt.DynQuantMatMulDequant(dX, dW, None, dS)
        rt.synchronize()
        aq, a_s, a_zp = oracle.dynamic_quantize_linear(c["X"])
        acc = oracle.matmul_integer(aq, c["W"], a_zp, None)
        want = oracle.dequant_epilogue(acc, a_s, c["w_scale"])
        assert np.array_equal(dq.numpy(), aq)
        assert np.array_equal(dacc.numpy(), acc)
        assert same_f32(dout.numpy(), want) and same_f32(dfused.numpy(), want)
    finally:
        rt.clear_cache()


# --------------------------------------------------------------------------
# full benchmark sizes: size-independent properties + sampled oracle rows
# --------------------------------------------------------------------------
@pytest.mark.parametrize("rows,cols", [(8192, 32768), (8191, 32767)])
def test_config2_full_size(rt, oracle, rows, cols):
    c = wl.config2(rows, cols)
    dX = rt.DeviceArray.from_numpy(c["X"])
    dS = rt.DeviceArray.from_numpy(c["scale"])
    dZ = rt.DeviceArray.from_numpy(c["zp"])
    dQ = rt.QuantizeLinear(dX, dS, dZ, axis=1)
    dD = rt.DequantizeLinear(dQ, dS, dZ, axis=1)
    dQ2 = rt.QuantizeLinear(dD, dS, dZ, axis=1)        # Q(DQ(q)) == q on the 8-bit lattice
    q = dQ.numpy()
    assert np.array_equal(q, dQ2.numpy())
    sample = np.r_[0:8, rows // 2:rows // 2 + 8, rows - 8:rows]
    want = oracle.quantize_linear(c["X"][sample], c["scale"], c["zp"], axis=1)
    assert np.array_equal(q[sample], want)
    d = dD.numpy()
    assert same_f32(d[sample], oracle.dequantize_linear(want, c["scale"], c["zp"], axis=1))
    # ... and every element against the oracle's OpenMP twin
    assert same_f32(d, oracle.dequantize_linear(q, c["scale"], c["zp"], axis=1, omp=True))
    del d, dD, dQ2
    # dynamic quantisation of the same tensor: parameters from numpy's min / max
    dY, ds, dz = rt.DynamicQuantizeLinear(dX)
    mn, mx = np.float32(min(c["X"].min(), 0)), np.float32(max(c["X"].max(), 0))
    s, zf, z = oracle.dynamic_params(float(c["X"].min()), float(c["X"].max()))
    assert ds.numpy().reshape(()) == s and int(dz.numpy().reshape(())) == int(z)
    y = dY.numpy()
    assert np.array_equal(y[sample], oracle.quantize_linear(c["X"][sample], s, np.array(z, np.uint8)))
    # per-tensor quantize / dequantize at full size against the oracle's OpenMP twin
    dQt = rt.QuantizeLinear(dX, np.float32(0.02), np.array(128, np.uint8))
    wq = oracle.quantize_linear(c["X"], np.float32(0.02), np.array(128, np.uint8), omp=True)
    assert np.array_equal(dQt.numpy(), wq)
