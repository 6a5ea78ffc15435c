"""Pins the CPU oracle before anything is compared with it.

Runs without a GPU.  Checks every function of oracle/om_oracle.c against
(a) the ONNX node-test vectors the reference enables, (b) answers held in the
reference's lit tests, (c) what the mathematics fixes: IEEE round-half-even,
brute force in Python integers on tiny shapes, algebraic identities chosen so
that a dropped term, a wrong sign or a transposed operand fails.
"""
import json
import math
import os

import numpy as np
import pytest

import oracle_lib

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "onnx_node_vectors.json")) as f:
    GOLD = json.load(f)


# ---------------------------------------------------------------- rounding --
def test_rne_matches_ieee_round_half_even(oracle):
    rng = np.random.default_rng(1)
    # every binade, exact ties, near-ties, huge, tiny, specials
    mant = rng.integers(0, 1 << 23, 4000, dtype=np.uint32)
    vals = []
    for e in range(0, 255, 3):
        bits = (np.uint32(e) << np.uint32(23)) | mant[:200]
        vals.append(bits.view(np.float32))
    ties = np.arange(-2000, 2000, dtype=np.float32) + np.float32(0.5)
    near = np.nextafter(ties, np.float32(np.inf)).astype(np.float32)
    near2 = np.nextafter(ties, np.float32(-np.inf)).astype(np.float32)
    v = np.concatenate(vals + [ties, near, near2, -np.concatenate(vals)[:3000],
                               np.array([0.0, -0.0, np.inf, -np.inf, 8388607.5, -8388607.5,
                                         16777216.0, 2.5, 3.5, -2.5, -3.5], np.float32)])
    want = np.rint(v)  # IEEE round-half-even in binary32
    got = np.array([oracle.rne(float(t)) for t in v], np.float32)
    assert np.array_equal(got, want)  # compares values; -0.0 == +0.0
    assert math.isnan(oracle.rne(float("nan")))


def test_rne_equals_rintf_for_every_binary32_value(oracle):
    """The floor-based round-half-even of the reference
    (src/Dialect/Mlir/DialectBuilder.cpp:291-332) against the C library's rintf
    on all 2^32 bit patterns (in C, all host threads; a few seconds)."""
    assert oracle.rne_sweep(0, 1 << 32) == 0


# ------------------------------------------------------------ golden: Q/DQ --
def test_quantizelinear_node_vector(oracle):
    g = GOLD["quantizelinear"]
    y = oracle.quantize_linear(np.array(g["x"], np.float32), np.float32(g["scale"]),
                               np.array(g["zp"], np.uint8))
    assert y.dtype == np.uint8 and y.tolist() == g["y"]


def test_quantizelinear_axis_spec_vector(oracle):
    # per-axis: parity unpinned by the reference (it asserts); ONNX spec vector only
    g = GOLD["quantizelinear_axis"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    y = oracle.quantize_linear(x, np.array(g["scale"], np.float32),
                               np.array(g["zp"], np.uint8), axis=g["axis"])
    assert y.reshape(-1).tolist() == g["y"]


def test_dequantizelinear_node_vector(oracle):
    g = GOLD["dequantizelinear"]
    y = oracle.dequantize_linear(np.array(g["x"], np.uint8), np.float32(g["scale"]),
                                 np.array(g["zp"], np.uint8))
    assert y.tolist() == g["y"]


def test_dequantizelinear_axis_spec_vector(oracle):
    g = GOLD["dequantizelinear_axis"]
    x = np.array(g["x"], np.uint8).reshape(g["x_shape"])
    y = oracle.dequantize_linear(x, np.array(g["scale"], np.float32),
                                 np.array(g["zp"], np.uint8), axis=g["axis"])
    assert y.reshape(-1).tolist() == g["y"]


@pytest.mark.parametrize("name", ["dynamicquantizelinear", "dynamicquantizelinear_max_adjusted",
                                  "dynamicquantizelinear_min_adjusted"])
def test_dynamicquantizelinear_node_vectors(oracle, name):
    g = GOLD[name]
    x = np.array(g["x"], np.float32)
    y, s, z = oracle.dynamic_quantize_linear(x)
    assert y.tolist() == g["y"]
    assert int(z) == g["zp"]
    assert s == np.float32(g["scale"])


def test_dynamic_params_edge_cases(oracle):
    # all-zero input: scale 0, 0/0 = NaN is dropped by maxnum -> zp 0, y 0
    y, s, z = oracle.dynamic_quantize_linear(np.zeros(7, np.float32))
    assert s == 0 and z == 0 and not y.any()
    # the zero point is saturated BEFORE it is rounded: min far below 0
    s, zf, z = oracle.dynamic_params(-10.0, 0.001)
    assert z == 255 and zf == 255.0
    # range is widened to include 0
    s, zf, z = oracle.dynamic_params(2.0, 4.0)
    assert z == 0 and s == np.float32(4.0) / np.float32(255.0)
    # NaN never wins a minnum / maxnum reduction
    mn, mx = oracle.minmax(np.array([np.nan, 1.0, -2.0, np.nan], np.float32))
    assert (mn, mx) == (-2.0, 1.0)


# ------------------------------------------ closed forms for quantize paths --
def _quant_exact(x, s, zp, lo, hi):
    """Same value through exact rational arithmetic where binary32 division is
    exact, i.e. power-of-two scales: round-half-even of x/s is then the
    mathematical one."""
    out = []
    for v in x:
        q = float(v) / float(s)          # exact for power-of-two s
        r = round(q)                      # Python rounds half to even
        out.append(int(min(max(r + zp, lo), hi)))
    return out


def test_quantize_matches_exact_arithmetic_for_pow2_scales(oracle):
    rng = np.random.default_rng(2)
    x = (rng.integers(-4000, 4000, 5000) / 8.0).astype(np.float32)  # many exact ties
    for s, zp, dt, lo, hi in [(0.25, 7, np.uint8, 0, 255), (2.0, -3, np.int8, -128, 127),
                              (0.5, 200, np.uint8, 0, 255)]:
        got = oracle.quantize_linear(x, np.float32(s), np.array(zp, dt))
        assert got.tolist() == _quant_exact(x, s, zp, lo, hi)
    # no zero point: output type defaults to uint8, nothing added
    got = oracle.quantize_linear(x, np.float32(0.5), None)
    assert got.tolist() == _quant_exact(x, 0.5, 0, 0, 255)


def test_quantize_uses_true_division_not_reciprocal(oracle):
    # x/s and x*(1/s) differ after rounding for these; the reference divides
    # unless --enable-fast-math (QuantizeLinear.cpp:43-44,129-132)
    s = np.float32(0.3)
    x = (np.arange(1, 20001, dtype=np.float32) * np.float32(0.15))
    d = np.rint(x / s)
    m = np.rint(x * (np.float32(1.0) / s))
    assert (d != m).any(), "sample does not separate divide from reciprocal"
    got = oracle.quantize_linear(x, s, None, out_dtype=np.uint8)
    want = np.clip(d, 0, 255).astype(np.uint8)
    assert np.array_equal(got, want)


def test_quantize_and_dql_under_the_two_compiler_options(oracle):
    """--enable-fast-math (x * (1 / scale), QuantizeLinear.cpp:43-44,119-132) and
    --disable-quantization-zero-point (QuantizeLinear.cpp:231-237,
    DynamicQuantizeLinear.cpp:75-84,142-152) against numpy's binary32
    arithmetic, on a sample where the reciprocal form and the divide differ
    within the unsaturated range (so taking one for the other fails), with a
    zero point that must be added in one mode and ignored in the other."""
    R, NZ = oracle_lib.RECIPROCAL, oracle_lib.NO_ZERO_POINT
    s = np.float32(0.3)
    x = np.concatenate([np.arange(1, 1601, dtype=np.float32) * np.float32(0.15),
                        -np.arange(1, 801, dtype=np.float32) * np.float32(0.15),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e30, 3e-39], np.float32)])
    r = np.float32(1.0) / s
    with np.errstate(all="ignore"):
        d, m = np.rint(x / s), np.rint(x * r)
    inside = (np.abs(d) < 120) & (d != m)
    assert inside.any(), "sample does not separate divide from reciprocal"

    def clip(v, dt):
        lo, hi = (0, 255) if dt == np.uint8 else (-128, 127)
        v = np.where(np.isnan(v), lo, v)          # maxnum then minnum: NaN -> lower bound
        return np.clip(v, lo, hi).astype(np.int64).astype(dt)

    for dt, zp in ((np.uint8, 7), (np.int8, -9)):
        z = np.array(zp, dt)
        for mode in (0, R, NZ, R | NZ):
            t = m if mode & R else d
            want = clip(t + (0 if mode & NZ else np.float32(zp)), dt)
            got = oracle.quantize_linear_mode(x, s, z, mode)
            assert got.dtype == dt and np.array_equal(got, want), (dt, mode)
        assert np.array_equal(oracle.quantize_linear_mode(x, s, z, 0), oracle.quantize_linear(x, s, z))
    # per-axis: scale[c], 1 / scale[c]
    xs = np.stack([x, x * 2], axis=1)
    sc = np.array([0.3, 0.7], np.float32)
    got = oracle.quantize_linear_mode(xs, sc, np.array([7, 3], np.uint8), R)
    with np.errstate(all="ignore"):
        want = np.stack([clip(np.rint(xs[:, c] * (np.float32(1) / sc[c])) + np.float32((7, 3)[c]), np.uint8)
                         for c in range(2)], axis=1)
    assert np.array_equal(got, want)
    # DynamicQuantizeLinear: the scale formula is untouched; the zero point is 0
    # and not added without zero points; the quotient by reciprocal with fast math
    rng = np.random.default_rng(95)
    for lo, hi in ((-3.0, 5.0), (0.5, 9.0), (-7.0, -1.0)):
        v = rng.uniform(lo, hi, 5000).astype(np.float32)
        y0, s0, z0 = oracle.dynamic_quantize_linear(v)
        for mode in (0, R, NZ, R | NZ):
            y, sc1, z = oracle.dynamic_quantize_linear_mode(v, mode)
            assert sc1 == s0
            zf = np.float32(0 if mode & NZ else z0)
            assert z == (0 if mode & NZ else z0)
            with np.errstate(all="ignore"):
                t = np.rint(v * (np.float32(1) / s0)) if mode & R else np.rint(v / s0)
            assert np.array_equal(y, clip(t + zf, np.uint8)), (lo, hi, mode)
        assert np.array_equal(oracle.dynamic_quantize_linear_mode(v, 0)[0], y0)


def test_quantize_special_values(oracle):
    x = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 0.0, -0.0], np.float32)
    y = oracle.quantize_linear(x, np.float32(0.1), np.array(10, np.uint8))
    assert y.tolist() == [0, 255, 0, 255, 0, 10, 10]   # NaN -> lower bound
    y = oracle.quantize_linear(x, np.float32(0.1), np.array(10, np.int8))
    assert y.tolist() == [-128, 127, -128, 127, -128, 10, 10]


def test_dequantize_closed_form_and_int32(oracle):
    rng = np.random.default_rng(3)
    x = rng.integers(-2**31, 2**31 - 1, 1000, dtype=np.int64).astype(np.int32)
    zp = np.array(12345, np.int32)
    s = np.float32(0.37)
    got = oracle.dequantize_linear(x, s, zp)
    want = (x.astype(np.float32) - np.float32(12345)) * s   # cast, sub, mul: three roundings
    assert np.array_equal(got, want)
    xi = rng.integers(-128, 128, 1000).astype(np.int8)
    got = oracle.dequantize_linear(xi, s, np.array(-7, np.int8))
    assert np.array_equal(got, (xi.astype(np.float32) + np.float32(7)) * s)
    got = oracle.dequantize_linear(xi, s, None)
    assert np.array_equal(got, xi.astype(np.float32) * s)


def test_quantize_dequantize_lattice_idempotence(oracle):
    # Q(DQ(q)) == q for every 8-bit q when the scale is a normal number
    q = np.arange(256, dtype=np.uint8)
    for s, zp in [(0.02, 128), (0.0051, 3), (1.7, 250)]:
        x = oracle.dequantize_linear(q, np.float32(s), np.array(zp, np.uint8))
        assert np.array_equal(oracle.quantize_linear(x, np.float32(s), np.array(zp, np.uint8)), q)


def test_per_axis_equals_per_tensor_slices(oracle):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 2, (3, 5, 4, 2)).astype(np.float32)
    for axis in range(4):
        C = x.shape[axis]
        sc = rng.uniform(0.005, 0.05, C).astype(np.float32)
        zp = rng.integers(0, 256, C).astype(np.uint8)
        y = oracle.quantize_linear(x, sc, zp, axis=axis)
        d = oracle.dequantize_linear(y, sc, zp, axis=axis)
        for c in range(C):
            sl = [slice(None)] * 4
            sl[axis] = c
            xs = np.ascontiguousarray(x[tuple(sl)])
            ys = oracle.quantize_linear(xs, sc[c], zp[c:c + 1])
            assert np.array_equal(y[tuple(sl)], ys)
            assert np.array_equal(d[tuple(sl)], oracle.dequantize_linear(ys, sc[c], zp[c:c + 1]))


def test_omp_variants_equal_scalar_ones(oracle):
    rng = np.random.default_rng(5)
    x = rng.normal(0, 2, (37, 53)).astype(np.float32)
    sc = rng.uniform(0.005, 0.05, 53).astype(np.float32)
    zp = rng.integers(0, 256, 53).astype(np.uint8)
    y = oracle.quantize_linear(x, sc, zp, axis=1)
    assert np.array_equal(y, oracle.quantize_linear(x, sc, zp, axis=1, omp=True))
    assert np.array_equal(oracle.dequantize_linear(y, sc, zp, axis=1),
                          oracle.dequantize_linear(y, sc, zp, axis=1, omp=True))
    a = oracle.dynamic_quantize_linear(x)
    b = oracle.dynamic_quantize_linear(x, omp=True)
    assert np.array_equal(a[0], b[0]) and a[1] == b[1] and a[2] == b[2]


# ------------------------------------------------------------ integer GEMMs --
def test_matmulinteger_node_vector(oracle):
    g = GOLD["matmulinteger"]
    y = oracle.matmul_integer(np.array(g["A"], np.uint8), np.array(g["B"], np.uint8),
                              np.array(g["a_zp"], np.uint8), np.array(g["b_zp"], np.uint8))
    assert y.tolist() == g["Y"]


def test_matmulinteger_constprop_answers(oracle):
    # test/mlir/onnx/onnx_constprop.mlir:1281-1289: ones[2,3] x ones[3,1] -> 3
    y = oracle.matmul_integer(np.ones((2, 3), np.int8), np.ones((3, 1), np.int8))
    assert y.tolist() == [[3], [3]]
    # :1179-1277: a matrix equal to its zero point gives an all-zero product for
    # scalar, per-row and per-column zero-point forms
    A = np.full((4, 3), 5, np.uint8)
    B = np.arange(6, dtype=np.uint8).reshape(3, 2)
    assert not oracle.matmul_integer(A, B, np.array(5, np.uint8), None).any()
    assert not oracle.matmul_integer(A, B, np.full(4, 5, np.uint8), np.array([1, 2], np.uint8)).any()
    Bc = np.tile(np.array([[7, 9]], np.uint8), (3, 1))
    assert not oracle.matmul_integer(B.T.copy(), Bc, None, np.array([7, 9], np.uint8)).any()


def _mmi_bruteforce(A, B, az, bz):
    M, K = A.shape
    N = B.shape[1]
    out = [[0] * N for _ in range(M)]
    for i in range(M):
        for j in range(N):
            acc = 0
            for k in range(K):
                a = int(A[i, k]) - (int(az[i]) if len(az) > 1 else (int(az[0]) if len(az) else 0))
                b = int(B[k, j]) - (int(bz[j]) if len(bz) > 1 else (int(bz[0]) if len(bz) else 0))
                acc += a * b
            acc = (acc + 2**31) % 2**32 - 2**31
            out[i][j] = acc
    return out


@pytest.mark.parametrize("adt,bdt", [(np.uint8, np.int8), (np.int8, np.uint8),
                                     (np.uint8, np.uint8), (np.int8, np.int8)])
def test_matmulinteger_bruteforce_small_shapes(oracle, adt, bdt):
    rng = np.random.default_rng(6)
    ia, ib = np.iinfo(adt), np.iinfo(bdt)
    for M in range(1, 6):
        for K in (1, 2, 7):
            for N in (1, 3, 8):
                A = rng.integers(ia.min, ia.max + 1, (M, K)).astype(adt)
                B = rng.integers(ib.min, ib.max + 1, (K, N)).astype(bdt)   # non-square: a transposed operand fails
                for az, bz in [([], []), ([int(ia.max)], [int(ib.min)]),
                               (rng.integers(ia.min, ia.max + 1, M).tolist(),
                                rng.integers(ib.min, ib.max + 1, N).tolist())]:
                    if len(az) == M == 1 or len(bz) == N == 1:
                        pass
                    got = oracle.matmul_integer(
                        A, B, np.array(az, adt) if az else None, np.array(bz, bdt) if bz else None)
                    assert got.tolist() == _mmi_bruteforce(A, B, az, bz)
                    got2 = oracle.matmul_integer(
                        A, B, np.array(az, adt) if az else None, np.array(bz, bdt) if bz else None,
                        passes=True)
                    assert np.array_equal(got, got2)


def test_matmulinteger_passes_matches_numpy_int64_mid_size(oracle):
    rng = np.random.default_rng(7)
    A = rng.integers(0, 256, (37, 129)).astype(np.uint8)
    B = rng.integers(-128, 128, (129, 45)).astype(np.int8)
    az = rng.integers(0, 256, 37).astype(np.uint8)
    bz = rng.integers(-128, 128, 45).astype(np.int8)
    want = (A.astype(np.int64) - az[:, None].astype(np.int64)) @ (B.astype(np.int64) - bz[None, :].astype(np.int64))
    want = ((want + 2**31) % 2**32 - 2**31).astype(np.int32)
    assert np.array_equal(oracle.matmul_integer(A, B, az, bz), want)
    assert np.array_equal(oracle.matmul_integer(A, B, az, bz, passes=True), want)


def test_qlinearmatmul_node_vectors(oracle):
    g = GOLD["qlinearmatmul_2D_uint8_float32"]
    a, b = np.array(g["a"], np.uint8), np.array(g["b"], np.uint8)
    acc = oracle.matmul_integer(a, b, np.array(g["a_zp"], np.uint8), np.array(g["b_zp"], np.uint8))
    assert acc.tolist() == g["acc"]
    for mode in (oracle_lib.WRAP, oracle_lib.SATURATE):   # the enabled node tests never saturate
        y = oracle.qlinear_matmul(a, g["a_scale"], np.array(g["a_zp"], np.uint8), b, g["b_scale"],
                                  np.array(g["b_zp"], np.uint8), g["y_scale"],
                                  np.array(g["y_zp"], np.uint8), mode)
        assert y.dtype == np.uint8 and y.tolist() == g["y"]
    g = GOLD["qlinearmatmul_2D_int8_float32"]
    a, b = np.array(g["a"], np.int8), np.array(g["b"], np.int8)
    for mode in (oracle_lib.WRAP, oracle_lib.SATURATE):
        y = oracle.qlinear_matmul(a, g["a_scale"], np.array(g["a_zp"], np.int8), b, g["b_scale"],
                                  np.array(g["b_zp"], np.int8), g["y_scale"],
                                  np.array(g["y_zp"], np.int8), mode)
        assert y.dtype == np.int8 and y.tolist() == g["y"]


def test_qlinearmatmul_wrap_vs_saturate_closed_form(oracle):
    # (roundEven(f32(acc)*s) + y_zp) mod 256 for wrap (trunci, QLinearMatMul.cpp:134-138),
    # clamped for saturate; the two agree exactly where 0 <= r + y_zp <= 255.
    rng = np.random.default_rng(8)
    a = rng.integers(0, 256, (9, 33)).astype(np.uint8)
    b = rng.integers(0, 256, (33, 11)).astype(np.uint8)
    az, bz, yz = np.array(128, np.uint8), np.array(120, np.uint8), np.array(0, np.uint8)
    acc = oracle.matmul_integer(a, b, az, bz)
    s = (np.float32(0.01) * np.float32(0.005)) / np.float32(0.002)
    r = np.rint(acc.astype(np.float32) * s).astype(np.int64) + int(yz)
    yw = oracle.qlinear_matmul(a, 0.01, az, b, 0.005, bz, 0.002, yz, oracle_lib.WRAP)
    ys = oracle.qlinear_matmul(a, 0.01, az, b, 0.005, bz, 0.002, yz, oracle_lib.SATURATE)
    assert np.array_equal(yw, (r % 256).astype(np.uint8))
    assert np.array_equal(ys, np.clip(r, 0, 255).astype(np.uint8))
    inside = (r >= 0) & (r <= 255)
    assert inside.any() and (~inside).any()
    assert np.array_equal(yw[inside], ys[inside]) and (yw[~inside] != ys[~inside]).mean() > 0.9
    # int8 output
    yzi = np.array(-5, np.int8)
    ai, bi = (a.astype(np.int16) - 128).astype(np.int8), (b.astype(np.int16) - 128).astype(np.int8)
    acc = oracle.matmul_integer(ai, bi, np.array(3, np.int8), np.array(-8, np.int8))
    r = np.rint(acc.astype(np.float32) * s).astype(np.int64) - 5
    yw = oracle.qlinear_matmul(ai, 0.01, np.array(3, np.int8), bi, 0.005, np.array(-8, np.int8), 0.002, yzi, oracle_lib.WRAP)
    ys = oracle.qlinear_matmul(ai, 0.01, np.array(3, np.int8), bi, 0.005, np.array(-8, np.int8), 0.002, yzi, oracle_lib.SATURATE)
    assert np.array_equal(yw, ((r + 128) % 256 - 128).astype(np.int8))
    assert np.array_equal(ys, np.clip(r, -128, 127).astype(np.int8))


def test_dequant_epilogue_closed_form(oracle):
    rng = np.random.default_rng(9)
    acc = rng.integers(-2**31, 2**31 - 1, (5, 7), dtype=np.int64).astype(np.int32)  # beyond 2^24: sitofp rounds
    bs = rng.uniform(1e-3, 1e-2, 7).astype(np.float32)
    a_s = np.float32(0.0313)
    want = acc.astype(np.float32) * (a_s * bs)[None, :]   # scale product first, then one multiply
    assert np.array_equal(oracle.dequant_epilogue(acc, a_s, bs), want)
    assert np.array_equal(oracle.dequant_epilogue(acc, a_s, bs[:1]), acc.astype(np.float32) * (a_s * bs[0]))


def test_batched_matmul_wrapper_equals_numpy_matmul(oracle):
    """The oracle handles a batched right-hand side by looping its 2-D routine
    over the batch entries that numpy's matmul rules pair up; the loop must
    reproduce numpy's own batched product (in int64, no wrap at these sizes)."""
    rng = np.random.default_rng(91)
    for ashape, bshape in (((2, 3, 5, 16), (2, 3, 16, 7)), ((3, 1, 4, 8), (5, 8, 6)), ((6, 8), (2, 8, 3)), ((8,), (2, 8, 3))):
        A = rng.integers(0, 256, ashape, dtype=np.uint8)
        B = rng.integers(-128, 128, bshape).astype(np.int8)
        az = np.array(rng.integers(0, 256), np.uint8)
        bz = rng.integers(-128, 128, bshape[:-2] + (1, bshape[-1])).astype(np.int8)
        want = np.matmul(A.astype(np.int64) - int(az), B.astype(np.int64) - bz.astype(np.int64))
        got = oracle.matmul_integer(A, B, az, bz)
        assert got.shape == want.shape and np.array_equal(got.astype(np.int64), want)



def test_relu_equals_numpy_fmax(oracle):
    """Relu is max(0, x) with the NaN rule of maxnum / fmax (the other operand
    wins): numpy's fmax is that operation.  Zeros compare equal whatever their
    sign, which the reference's operation leaves open."""
    rng = np.random.default_rng(92)
    x = rng.standard_normal(10000).astype(np.float32)
    x[:8] = [np.nan, -np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-45, -1e-45]
    got = oracle.relu(x)
    assert np.array_equal(got, np.fmax(x, np.float32(0)))
    assert got[0] == 0 and got[1] == 0 and got[2] == np.inf and got[3] == 0
    assert not np.signbit(got[5]) and got[6] == np.float32(1e-45)


def test_gelu_is_the_erf_formula(oracle):
    """Gelu (approximate "none") against 0.5 x (1 + erf(x / sqrt 2)) evaluated
    in binary64: pins the formula (a dropped 0.5, sqrt 2 for 1 / sqrt 2 or erf
    for 1 + erf is off by far more than the bound), not the last bits, which
    depend on whose erf is used.  Bound: one unit in the last place of erf
    times |0.5 x|, plus the roundings of the products."""
    from math import erf, sqrt
    rng = np.random.default_rng(93)
    x = np.concatenate([rng.standard_normal(20000) * 3, np.linspace(-9, 9, 2001),
                        [0.0, -0.0, 1e-30, -1e-30, 40.0, -40.0]]).astype(np.float32)
    got = oracle.gelu(x).astype(np.float64)
    x64 = x.astype(np.float64)
    want = np.array([0.5 * v * (1.0 + erf(v / sqrt(2.0))) for v in x64])
    tol = np.abs(0.5 * x64) * 2.0 ** -23 + np.abs(want) * 2.0 ** -22 + 1e-45
    assert (np.abs(got - want) <= tol).all()
    assert got[-2] == 40.0 and got[-1] == 0.0
    special = oracle.gelu(np.array([np.inf, -np.inf, np.nan], np.float32))
    # 0.5 * -inf * (1 + -1) = -inf * 0 is a NaN, as the formula gives it
    assert special[0] == np.inf and np.isnan(special[1]) and np.isnan(special[2])


def test_four_instruction_quotient_equals_the_divide(tmp_path):
    """The quantize kernels divide by a scale of ordinary magnitude with a
    reciprocal multiply and one exact correction step.  tests/quotient_check.c
    restates that sequence on the CPU (fmaf is the GPU's v_fma_f32) and compares
    it with the IEEE divide: bit for bit where the quotient matters (random pairs,
    and every neighbour of a half-integer or integer quotient for thousands of
    scales), and through the 8-bit result for arbitrary x (tiny, huge, infinite,
    NaN).  Half a billion pairs, a few seconds on all host threads."""
    import shutil, subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    exe = str(tmp_path / "quotient_check")
    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quotient_check.c")
    subprocess.check_call(["gcc", "-O2", "-march=x86-64-v3", "-fopenmp", "-ffp-contract=off", "-o", exe, src, "-lm"])
    out = subprocess.run([exe, "20000000", "20000"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "0 quotients differ, 0 8-bit results differ" in out.stdout
