"""ctypes binding of the CPU oracle (oracle/libom_oracle.so) for the tests.

The oracle is the checker only: the product never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libom_oracle.so")

U8, I8, I32 = 0, 1, 2
WRAP, SATURATE = 0, 1
RECIPROCAL, NO_ZERO_POINT = 1, 2   # bits of `mode` (compiler options that change the arithmetic)

_KIND = {np.dtype(np.uint8): U8, np.dtype(np.int8): I8, np.dtype(np.int32): I32}


def kind_of(a) -> int:
    return _KIND[np.dtype(a.dtype)]


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        P, I64, F, I = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int
        lib.om_oracle_rne.restype = F
        lib.om_oracle_rne.argtypes = [F]
        lib.om_oracle_rne_sweep.restype = I64
        lib.om_oracle_rne_sweep.argtypes = [ctypes.c_uint32, I64]
        for name in ("om_oracle_quantize_linear", "om_oracle_quantize_linear_omp"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [P, I64, I64, I64, P, P, I, P]
        for name in ("om_oracle_dequantize_linear", "om_oracle_dequantize_linear_omp"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [P, I, I64, I64, I64, P, P, P]
        lib.om_oracle_minmax.restype = None
        lib.om_oracle_minmax.argtypes = [P, I64, P, P]
        lib.om_oracle_dynamic_params.restype = None
        lib.om_oracle_dynamic_params.argtypes = [F, F, P, P, P]
        for name in ("om_oracle_dynamic_quantize_linear", "om_oracle_dynamic_quantize_linear_omp"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [P, I64, P, P, P]
        lib.om_oracle_quantize_linear_mode.restype = None
        lib.om_oracle_quantize_linear_mode.argtypes = [P, I64, I64, I64, P, P, I, P, I]
        lib.om_oracle_dynamic_quantize_linear_mode.restype = None
        lib.om_oracle_dynamic_quantize_linear_mode.argtypes = [P, I64, P, P, P, I]
        for name in ("om_oracle_matmul_integer", "om_oracle_matmul_integer_passes"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [P, I, P, I, I64, I64, I64, P, I64, P, I64, P]
        lib.om_oracle_qlinear_matmul.restype = None
        lib.om_oracle_qlinear_matmul.argtypes = [
            P, I, F, P, I64, P, I, F, P, I64, F, P, I, I64, I64, I64, I, P]
        lib.om_oracle_dequant_epilogue.restype = None
        lib.om_oracle_dequant_epilogue.argtypes = [P, I64, I64, F, P, I64, P]
        lib.om_oracle_relu.restype = None
        lib.om_oracle_relu.argtypes = [P, I64, P]
        lib.om_oracle_gelu.restype = None
        lib.om_oracle_gelu.argtypes = [P, I64, P]
        lib.om_oracle_num_threads.restype = I

    # -- helpers ----------------------------------------------------------
    @staticmethod
    def _split(shape, scale, axis):
        n = int(np.prod(shape, dtype=np.int64))
        if scale.size == 1:
            return 1, 1, n
        axis = axis % len(shape)
        outer = int(np.prod(shape[:axis], dtype=np.int64))
        inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
        assert shape[axis] == scale.size
        return outer, scale.size, inner

    def rne_sweep(self, first_bits: int, count: int) -> int:
        return int(self.lib.om_oracle_rne_sweep(first_bits, count))

    def rne(self, x: float) -> float:
        return float(self.lib.om_oracle_rne(ctypes.c_float(x)))

    def quantize_linear(self, x, scale, zp=None, axis=1, out_dtype=np.uint8, omp=False):
        x = np.ascontiguousarray(x, np.float32)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        if zp is not None:
            zp = np.ascontiguousarray(zp).reshape(-1)
            out_dtype = zp.dtype
        y = np.empty(x.shape, out_dtype)
        outer, ch, inner = self._split(x.shape, scale, axis)
        fn = self.lib.om_oracle_quantize_linear_omp if omp else self.lib.om_oracle_quantize_linear
        fn(_p(x), outer, ch, inner, _p(scale), _p(zp), _KIND[np.dtype(out_dtype)], _p(y))
        return y

    def quantize_linear_mode(self, x, scale, zp, mode, axis=1, out_dtype=np.uint8):
        """QuantizeLinear as compiled with the options in `mode` (RECIPROCAL |
        NO_ZERO_POINT); the output type still follows the zero point's."""
        x = np.ascontiguousarray(x, np.float32)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        if zp is not None:
            zp = np.ascontiguousarray(zp).reshape(-1)
            out_dtype = zp.dtype
        y = np.empty(x.shape, out_dtype)
        outer, ch, inner = self._split(x.shape, scale, axis)
        self.lib.om_oracle_quantize_linear_mode(_p(x), outer, ch, inner, _p(scale), _p(zp),
                                                _KIND[np.dtype(out_dtype)], _p(y), int(mode))
        return y

    def dynamic_quantize_linear_mode(self, x, mode):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(x.shape, np.uint8)
        s, z = ctypes.c_float(), ctypes.c_uint8()
        self.lib.om_oracle_dynamic_quantize_linear_mode(_p(x), x.size, _p(y), ctypes.byref(s),
                                                        ctypes.byref(z), int(mode))
        return y, np.float32(s.value), np.uint8(z.value)

    def dequantize_linear(self, x, scale, zp=None, axis=1, omp=False):
        x = np.ascontiguousarray(x)
        scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
        if zp is not None:
            zp = np.ascontiguousarray(zp).reshape(-1)
            assert zp.dtype == x.dtype
        y = np.empty(x.shape, np.float32)
        outer, ch, inner = self._split(x.shape, scale, axis)
        fn = self.lib.om_oracle_dequantize_linear_omp if omp else self.lib.om_oracle_dequantize_linear
        fn(_p(x), kind_of(x), outer, ch, inner, _p(scale), _p(zp), _p(y))
        return y

    def minmax(self, x):
        x = np.ascontiguousarray(x, np.float32)
        mn, mx = ctypes.c_float(), ctypes.c_float()
        self.lib.om_oracle_minmax(_p(x), x.size, ctypes.byref(mn), ctypes.byref(mx))
        return mn.value, mx.value

    def dynamic_params(self, xmin, xmax):
        s, zf, z = ctypes.c_float(), ctypes.c_float(), ctypes.c_uint8()
        self.lib.om_oracle_dynamic_params(ctypes.c_float(xmin), ctypes.c_float(xmax),
                                          ctypes.byref(s), ctypes.byref(zf), ctypes.byref(z))
        return np.float32(s.value), np.float32(zf.value), np.uint8(z.value)

    def dynamic_quantize_linear(self, x, omp=False):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(x.shape, np.uint8)
        s, z = ctypes.c_float(), ctypes.c_uint8()
        fn = (self.lib.om_oracle_dynamic_quantize_linear_omp if omp
              else self.lib.om_oracle_dynamic_quantize_linear)
        fn(_p(x), x.size, _p(y), ctypes.byref(s), ctypes.byref(z))
        return y, np.float32(s.value), np.uint8(z.value)

    @staticmethod
    def _batched(a, b, a_zp, b_zp):
        """Splits a product with a batched right-hand side into its 2-D
        products, as numpy's matmul broadcasts them: yields (index of the result
        matrix, A matrix, B matrix, a_zp for it, b_zp for it).  Zero points of
        the forms [.., M, 1] / [.., 1, N] are sliced along with their matrix."""
        a2 = a if a.ndim >= 2 else a.reshape(1, -1)
        batch = np.broadcast_shapes(a2.shape[:-2], b.shape[:-2])
        ab = np.broadcast_to(a2, batch + a2.shape[-2:])
        bb = np.broadcast_to(b, batch + b.shape[-2:])
        azb = bzb = None
        if a_zp is not None and np.ndim(a_zp) > 1:
            azb = np.broadcast_to(np.asarray(a_zp), batch + (a2.shape[-2], 1))
        if b_zp is not None and np.ndim(b_zp) > 1:
            bzb = np.broadcast_to(np.asarray(b_zp), batch + (1, b.shape[-1]))
        for idx in np.ndindex(*batch):
            yield (idx, np.ascontiguousarray(ab[idx]), np.ascontiguousarray(bb[idx]),
                   a_zp if azb is None else np.ascontiguousarray(azb[idx]).reshape(-1),
                   b_zp if bzb is None else np.ascontiguousarray(bzb[idx]).reshape(-1))

    def matmul_integer(self, a, b, a_zp=None, b_zp=None, passes=False):
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        if b.ndim > 2:     # one 2-D product per batch entry
            batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
            rows = (a.shape[-2],) if a.ndim >= 2 else ()
            y = np.empty(batch + rows + (b.shape[-1],), np.int32)
            for idx, am, bm, az, bz in self._batched(a, b, a_zp, b_zp):
                y[idx] = self.matmul_integer(am, bm, az, bz, passes).reshape(y[idx].shape)
            return y
        if b.ndim == 1:
            return self.matmul_integer(a, b.reshape(-1, 1), a_zp, b_zp, passes)[..., 0]
        K, N = b.shape
        M = a.size // K if K else int(np.prod(a.shape[:-1]))
        az = None if a_zp is None else np.ascontiguousarray(a_zp, a.dtype).reshape(-1)
        bz = None if b_zp is None else np.ascontiguousarray(b_zp, b.dtype).reshape(-1)
        y = np.empty(tuple(a.shape[:-1]) + (N,), np.int32)
        fn = self.lib.om_oracle_matmul_integer_passes if passes else self.lib.om_oracle_matmul_integer
        fn(_p(a), kind_of(a), _p(b), kind_of(b), M, K, N, _p(az), 0 if az is None else az.size,
           _p(bz), 0 if bz is None else bz.size, _p(y))
        return y

    def qlinear_matmul(self, a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, mode=WRAP):
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        if b.ndim > 2:
            batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
            rows = (a.shape[-2],) if a.ndim >= 2 else ()
            y = np.empty(batch + rows + (b.shape[-1],), np.asarray(y_zp).dtype)
            for idx, am, bm, az, bz in self._batched(a, b, a_zp, b_zp):
                y[idx] = self.qlinear_matmul(am, a_scale, az, bm, b_scale, bz, y_scale, y_zp,
                                             mode).reshape(y[idx].shape)
            return y
        K, N = b.shape
        M = a.size // K if K else int(np.prod(a.shape[:-1]))
        az = np.ascontiguousarray(a_zp, a.dtype).reshape(-1)
        bz = np.ascontiguousarray(b_zp, b.dtype).reshape(-1)
        yz = np.ascontiguousarray(y_zp).reshape(-1)
        y = np.empty(tuple(a.shape[:-1]) + (N,), yz.dtype)
        f = lambda v: ctypes.c_float(float(np.float32(np.asarray(v).reshape(-1)[0])))
        self.lib.om_oracle_qlinear_matmul(
            _p(a), kind_of(a), f(a_scale), _p(az), az.size, _p(b), kind_of(b), f(b_scale),
            _p(bz), bz.size, f(y_scale), _p(yz), kind_of(yz), M, K, N, mode, _p(y))
        return y

    def dequant_epilogue(self, acc, a_scale, b_scale):
        acc = np.ascontiguousarray(acc, np.int32)
        bs = np.ascontiguousarray(b_scale, np.float32).reshape(-1)
        N = acc.shape[-1]
        M = acc.size // N
        out = np.empty(acc.shape, np.float32)
        self.lib.om_oracle_dequant_epilogue(
            _p(acc), M, N, ctypes.c_float(float(np.float32(a_scale))), _p(bs), bs.size, _p(out))
        return out

    def relu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.float32)
        self.lib.om_oracle_relu(_p(x), x.size, _p(out))
        return out

    def gelu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty(x.shape, np.float32)
        self.lib.om_oracle_gelu(_p(x), x.size, _p(out))
        return out

    def num_threads(self):
        return int(self.lib.om_oracle_num_threads())


_oracle = None


def load() -> Oracle:
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "all"])
        _oracle = Oracle(ctypes.CDLL(ORACLE_SO))
    return _oracle
