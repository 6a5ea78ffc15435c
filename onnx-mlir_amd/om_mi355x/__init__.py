"""Host-side binding of the MI355X runtime for onnx-mlir's int8 path.

The functions mirror the ONNX operators the reference lowers on its CPU path
(QuantizeLinear, DequantizeLinear, DynamicQuantizeLinear, MatMulInteger,
QLinearMatMul; src/Conversion/ONNXToKrnl/ConvertONNXToKrnl.cpp:226-241) and
call the C-ABI entry points of ``include/om_mi355x.h`` exactly as a compiled
model's ``krnl.call`` would: outputs first, then inputs, then integer
attributes, every tensor wrapped in an ``OMTensor``
(src/Conversion/KrnlToLLVM/KrnlCall.cpp:34-102).

Operands may be numpy arrays (host memory: the runtime stages them through the
GPU and copies results back) or :class:`DeviceArray` (GPU memory owned by the
runtime: used in place, results stay on the GPU).

There is no CPU implementation here.  If the HIP library is missing or no
gfx950 device is present the calls raise.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence, Tuple, Union

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.normpath(os.path.join(_HERE, "..", "csrc"))
LIB_PATH = os.path.join(_CSRC, "libom_mi355x.so")
SHIM_PATH = os.path.join(_CSRC, "libom_tensor_shim.so")
# measurement aids (csrc/measure), outside the runtime's C-ABI
MEASURE_PATH = os.path.join(_CSRC, "libom_mi355x_measure.so")

# ONNX element-type codes (include/onnx-mlir/Runtime/OnnxDataTypeMetaData.inc:22-44)
ONNX_FLOAT, ONNX_UINT8, ONNX_INT8, ONNX_INT32 = 1, 2, 3, 6
_NP_TO_ONNX = {
    np.dtype(np.float32): ONNX_FLOAT,
    np.dtype(np.uint8): ONNX_UINT8,
    np.dtype(np.int8): ONNX_INT8,
    np.dtype(np.int32): ONNX_INT32,
}

WRAP, SATURATE = 0, 1
# `activation` of the fused entry points (OM_MI355X_ACTIVATION_* of the header)
ACTIVATION_NONE, ACTIVATION_RELU, ACTIVATION_GELU = 0, 1, 2
# bits of set_quant_mode (OM_MI355X_QUANT_* of the header): the reference's
# --enable-fast-math and --disable-quantization-zero-point
QUANT_RECIPROCAL, QUANT_NO_ZERO_POINT = 1, 2
# OM_MI355X_VERSION of the header this module was written against
VERSION = 0x00010100


class RuntimeError_(RuntimeError):
    """An entry point reported an error (errno + message)."""


_lib = None
_shim = None


def library_present() -> bool:
    return os.path.exists(LIB_PATH) and os.path.exists(SHIM_PATH)


def load(tensor_runtime: Optional[str] = None):
    """Load the runtime.  ``tensor_runtime`` names an alternative provider of
    the ``omTensor*`` accessors (e.g. the reference's own C runtime); it is
    loaded with RTLD_GLOBAL first so that it wins symbol resolution."""
    global _lib, _shim
    if _lib is not None:
        return _lib
    if not library_present():
        raise FileNotFoundError(
            f"{LIB_PATH} is not built; run __graft_entry__.build() "
            "(make -C onnx-mlir_amd/csrc)")
    provider = tensor_runtime or SHIM_PATH
    _shim = ctypes.CDLL(provider, mode=ctypes.RTLD_GLOBAL)
    _lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    _declare(_lib, _shim)
    return _lib


def _declare(lib, shim):
    P, I64, SZ = ctypes.c_void_p, ctypes.c_int64, ctypes.c_size_t
    shim.omTensorCreate.restype = P
    shim.omTensorCreate.argtypes = [P, ctypes.POINTER(I64), I64, ctypes.c_int]
    shim.omTensorDestroy.restype = None
    shim.omTensorDestroy.argtypes = [P]
    sigs = {
        "om_mi355x_QuantizeLinear": [P, P, P, P, I64, I64],
        "om_mi355x_DequantizeLinear": [P, P, P, P, I64],
        "om_mi355x_DynamicQuantizeLinear": [P, P, P, P],
        "om_mi355x_DynamicQuantizeLinearNoAlloc": [P, P, P, P],
        "om_mi355x_MatMulInteger": [P, P, P, P, P],
        "om_mi355x_MatMulIntegerDequant": [P, P, P, P, P, P, P, P, I64],
        "om_mi355x_QLinearMatMul": [P, P, P, P, P, P, P, P, P, I64],
        "om_mi355x_DynQuantMatMulDequant": [P, P, P, P, P, P, I64],
        "om_mi355x_DynQuantMatMulDequantLimits": [P, P, P, P, P, P, P, P, I64],
        "om_mi355x_MarkConstant": [P],
        "om_mi355x_UnmarkConstant": [P],
        "om_mi355x_KeepOnDevice": [P],
        "om_mi355x_Release": [P],
        "om_mi355x_ClearCache": [],
        "OMInitAccelMI355X": [],
        "OMShutdownAccelMI355X": [],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.restype = None
        fn.argtypes = args
    lib.OMInitCompatibleAccelMI355X.restype = ctypes.c_uint64
    lib.OMInitCompatibleAccelMI355X.argtypes = [ctypes.c_uint64]
    lib.om_mi355x_malloc.restype = P
    lib.om_mi355x_malloc.argtypes = [SZ]
    lib.om_mi355x_free.restype = None
    lib.om_mi355x_free.argtypes = [P]
    lib.om_mi355x_memcpy_h2d.restype = ctypes.c_int
    lib.om_mi355x_memcpy_h2d.argtypes = [P, P, SZ]
    lib.om_mi355x_memcpy_d2h.restype = ctypes.c_int
    lib.om_mi355x_memcpy_d2h.argtypes = [P, P, SZ]
    lib.om_mi355x_synchronize.restype = ctypes.c_int
    lib.om_mi355x_timer_start.restype = ctypes.c_int
    lib.om_mi355x_timer_stop.restype = ctypes.c_float
    lib.om_mi355x_last_error.restype = ctypes.c_char_p
    lib.om_mi355x_last_gemm_kernel.restype = ctypes.c_char_p
    lib.om_mi355x_device_info.restype = ctypes.c_int
    lib.om_mi355x_SetQuantMode.restype = None
    lib.om_mi355x_SetQuantMode.argtypes = [ctypes.c_void_p, ctypes.c_int64]
    lib.om_mi355x_GetQuantMode.restype = ctypes.c_int64
    lib.om_mi355x_device_info.argtypes = [ctypes.c_char_p, SZ]


def _check():
    msg = _lib.om_mi355x_last_error()
    if msg:
        raise RuntimeError_(msg.decode())


def device_info() -> dict:
    load()
    buf = ctypes.create_string_buffer(256)
    if _lib.om_mi355x_device_info(buf, 256) != 0:
        _check()
        raise RuntimeError_("no device")
    name, arch, cus, mhz, gib = buf.value.decode().split("|")
    return {"name": name, "arch": arch, "cus": int(cus), "clock_mhz": int(mhz),
            "mem_gib": float(gib)}


# The compiler options this binding "compiles" its calls with.  In the runtime
# the mode belongs to one op (om_mi355x_SetQuantMode applies to the thread's
# next quantize / dequantize / dynamic-quantize / fused-layer call only), so
# the binding does what generated code does: while the mode is non-zero it puts
# om_mi355x_SetQuantMode in front of each such call, and nothing otherwise.
_compiled_mode = 0


def set_quant_mode(mode: int) -> None:
    """How the QuantizeLinear / DequantizeLinear / DynamicQuantizeLinear calls
    (and the whole-layer fused call) made through this module from now on
    compute: 0 as the reference does by default, or QUANT_RECIPROCAL |
    QUANT_NO_ZERO_POINT as it does when compiled with --enable-fast-math /
    --disable-quantization-zero-point."""
    global _compiled_mode
    load()
    _lib.om_mi355x_SetQuantMode(None, ctypes.c_int64(int(mode)))   # validates
    _check()
    _lib.om_mi355x_SetQuantMode(None, ctypes.c_int64(0))
    _compiled_mode = int(mode)


def quant_mode() -> int:
    return _compiled_mode


def pending_quant_mode() -> int:
    """The mode the calling thread's next such op would take in the runtime
    (om_mi355x_GetQuantMode): non-zero only between om_mi355x_SetQuantMode and
    the op it precedes."""
    load()
    return int(_lib.om_mi355x_GetQuantMode())


def _emit_quant_mode():
    if _compiled_mode:
        _lib.om_mi355x_SetQuantMode(None, ctypes.c_int64(_compiled_mode))


_measure = None


def mfma_ceiling(random_operands: bool = True) -> dict:
    """int8 MFMA rate of the device with nothing else going on (TOPS) and the
    shader clock it held meanwhile (csrc/measure/mfma_ceiling.h; a library of
    its own, not part of the runtime)."""
    global _measure
    if _measure is None:
        _measure = ctypes.CDLL(MEASURE_PATH)
        _measure.om_mi355x_measure_mfma_ceiling.restype = ctypes.c_int
        _measure.om_mi355x_measure_mfma_ceiling.argtypes = [
            ctypes.c_int64, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    tops, ghz = ctypes.c_double(0.0), ctypes.c_double(0.0)
    rc = _measure.om_mi355x_measure_mfma_ceiling(ctypes.c_int64(1 if random_operands else 0),
                                                 ctypes.byref(tops), ctypes.byref(ghz))
    if rc != 0:
        raise RuntimeError_(f"om_mi355x_measure_mfma_ceiling failed: HIP error {rc}")
    return {"tops": tops.value, "clock_ghz": ghz.value}


def last_gemm_kernel() -> str:
    """Name of the GEMM kernel this thread's last matmul call launched."""
    load()
    return _lib.om_mi355x_last_gemm_kernel().decode()


def init_compatible(version: int = VERSION) -> bool:
    load()
    return bool(_lib.OMInitCompatibleAccelMI355X(version))


class DeviceArray:
    """A row-major tensor in GPU memory obtained from the runtime."""

    def __init__(self, shape: Sequence[int], dtype):
        load()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self.ptr = _lib.om_mi355x_malloc(max(self.nbytes, 16))
        if not self.ptr:
            _check()
            raise MemoryError("om_mi355x_malloc failed")

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceArray":
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        if a.nbytes and _lib.om_mi355x_memcpy_h2d(
                d.ptr, a.ctypes.data_as(ctypes.c_void_p), a.nbytes) != 0:
            _check()
        return d

    @classmethod
    def view_of(cls, owner: "DeviceArray", offset_elems: int, shape) -> "DeviceArray":
        """A window into ``owner``'s memory starting ``offset_elems`` elements in."""
        v = cls.__new__(cls)
        v.shape = tuple(int(s) for s in shape)
        v.dtype = owner.dtype
        v.size = int(np.prod(v.shape, dtype=np.int64)) if v.shape else 1
        v.nbytes = v.size * v.dtype.itemsize
        assert offset_elems * v.dtype.itemsize + v.nbytes <= owner.nbytes
        v.ptr = owner.ptr + offset_elems * v.dtype.itemsize
        v.owner = owner
        return v

    def numpy(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        if self.nbytes and _lib.om_mi355x_memcpy_d2h(
                out.ctypes.data_as(ctypes.c_void_p), self.ptr, self.nbytes) != 0:
            _check()
        return out

    def free(self):
        if getattr(self, "owner", None) is not None:
            self.ptr = None
            return
        if self.ptr:
            _lib.om_mi355x_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


Tensor = Union[np.ndarray, DeviceArray]


class _OMT:
    """A non-owning OMTensor wrapper around a numpy array or DeviceArray, made
    the way the generated code makes one per krnl.call operand."""

    def __init__(self, t: Optional[Tensor]):
        self.handle = None
        self.keep = t
        if t is None:
            return
        if isinstance(t, DeviceArray):
            ptr, shape, dt = t.ptr, t.shape, t.dtype
        else:
            if not t.flags["C_CONTIGUOUS"]:
                raise ValueError("host tensors must be C-contiguous")
            ptr, shape, dt = t.ctypes.data, t.shape, t.dtype
        code = _NP_TO_ONNX.get(np.dtype(dt))
        if code is None:
            raise TypeError(f"unsupported element type {dt}")
        arr = (ctypes.c_int64 * max(len(shape), 1))(*shape)
        self.handle = _shim.omTensorCreate(ptr, arr, len(shape), code)
        if not self.handle:
            raise MemoryError("omTensorCreate failed")

    def __enter__(self):
        return self.handle

    def __exit__(self, *exc):
        if self.handle:
            _shim.omTensorDestroy(self.handle)
            self.handle = None


def _like(template: Tensor, shape, dtype) -> Tensor:
    if isinstance(template, DeviceArray):
        return DeviceArray(shape, dtype)
    return np.empty(shape, dtype)


def _host(a, dtype=None) -> Tensor:
    if isinstance(a, DeviceArray):
        return a
    a = np.asarray(a) if dtype is None else np.asarray(a, dtype=dtype)
    return np.ascontiguousarray(a)


# Arrays declared constant, by data address: the runtime keys its caches by
# that address, so the array must stay alive (and its address taken) until
# unmark_constant or clear_cache.
_marked = {}


def mark_constant(t: Tensor):
    """Declare that ``t`` never changes (a model constant).  The binding keeps
    ``t`` alive until :func:`unmark_constant` or :func:`clear_cache`."""
    load()
    with _OMT(t) as h:
        _lib.om_mi355x_MarkConstant(h)
    _marked[t.ptr if isinstance(t, DeviceArray) else t.ctypes.data] = t


def unmark_constant(t: Tensor):
    """Take the declaration back and drop what the runtime cached for ``t``."""
    load()
    with _OMT(t) as h:
        _lib.om_mi355x_UnmarkConstant(h)
    _marked.pop(t.ptr if isinstance(t, DeviceArray) else t.ctypes.data, None)


def clear_cache():
    load()
    _lib.om_mi355x_ClearCache()
    _marked.clear()


def keep_on_device(t: np.ndarray):
    """Back the host buffer of ``t`` with GPU memory: until ``release`` the ops
    use that memory whenever they are handed ``t`` and never touch the host
    buffer (what a compiled model does for results that only feed other
    offloaded ops)."""
    load()
    with _OMT(t) as h:
        _lib.om_mi355x_KeepOnDevice(h)
    _check()


def release(t: np.ndarray):
    load()
    with _OMT(t) as h:
        _lib.om_mi355x_Release(h)
    _check()


def synchronize():
    load()
    if _lib.om_mi355x_synchronize() != 0:
        _check()


def timer_start():
    if _lib.om_mi355x_timer_start() != 0:
        _check()


def timer_stop() -> float:
    ms = float(_lib.om_mi355x_timer_stop())
    if ms < 0:
        _check()
    return ms


def QuantizeLinear(x: Tensor, y_scale: Tensor, y_zero_point: Optional[Tensor] = None,
                   axis: int = 1, saturate: int = 1, out: Optional[Tensor] = None) -> Tensor:
    load()
    x, y_scale = _host(x), _host(y_scale, np.float32)
    ydt = np.uint8 if y_zero_point is None else _host(y_zero_point).dtype
    if y_zero_point is not None:
        y_zero_point = _host(y_zero_point)
    y = out if out is not None else _like(x, x.shape, ydt)
    with _OMT(y) as hy, _OMT(x) as hx, _OMT(y_scale) as hs, _OMT(y_zero_point) as hz:
        _emit_quant_mode()
        _lib.om_mi355x_QuantizeLinear(hy, hx, hs, hz, axis, saturate)
    _check()
    return y


def DequantizeLinear(x: Tensor, x_scale: Tensor, x_zero_point: Optional[Tensor] = None,
                     axis: int = 1, out: Optional[Tensor] = None) -> Tensor:
    load()
    x, x_scale = _host(x), _host(x_scale, np.float32)
    if x_zero_point is not None:
        x_zero_point = _host(x_zero_point)
    y = out if out is not None else _like(x, x.shape, np.float32)
    with _OMT(y) as hy, _OMT(x) as hx, _OMT(x_scale) as hs, _OMT(x_zero_point) as hz:
        _emit_quant_mode()
        _lib.om_mi355x_DequantizeLinear(hy, hx, hs, hz, axis)
    _check()
    return y


def DynamicQuantizeLinear(x: Tensor, out: Optional[Tuple[Tensor, Tensor, Tensor]] = None
                          ) -> Tuple[Tensor, Tensor, Tensor]:
    load()
    x = _host(x)
    if out is not None:
        y, s, z = out
    else:
        y = _like(x, x.shape, np.uint8)
        s = _like(x, (), np.float32)
        z = _like(x, (), np.uint8)
    with _OMT(y) as hy, _OMT(s) as hs, _OMT(z) as hz, _OMT(x) as hx:
        _emit_quant_mode()
        _lib.om_mi355x_DynamicQuantizeLinear(hy, hs, hz, hx)
    _check()
    return y, s, z


def DynamicQuantizeLinearNoAlloc(x: DeviceArray, out: Tuple[DeviceArray, DeviceArray, DeviceArray]
                                 ) -> Tuple[DeviceArray, DeviceArray, DeviceArray]:
    """DynamicQuantizeLinear through the entry point that allocates nothing: all
    four tensors are GPU memory the caller allocated beforehand."""
    load()
    y, s, z = out
    with _OMT(y) as hy, _OMT(s) as hs, _OMT(z) as hz, _OMT(x) as hx:
        _emit_quant_mode()
        _lib.om_mi355x_DynamicQuantizeLinearNoAlloc(hy, hs, hz, hx)
    _check()
    return y, s, z


def _mm_shape(a: Tensor, b: Tensor):
    """Result shape of onnx.MatMul(a, b) (numpy's matmul rules)."""
    if len(b.shape) == 1:
        return tuple(a.shape[:-1])
    if len(b.shape) == 2:
        return tuple(a.shape[:-1]) + (b.shape[-1],)
    batch = np.broadcast_shapes(tuple(a.shape[:-2]), tuple(b.shape[:-2]))
    rows = (a.shape[-2],) if len(a.shape) >= 2 else ()
    return tuple(batch) + rows + (b.shape[-1],)


def MatMulInteger(a: Tensor, b: Tensor, a_zero_point: Optional[Tensor] = None,
                  b_zero_point: Optional[Tensor] = None, out: Optional[Tensor] = None) -> Tensor:
    load()
    a, b = _host(a), _host(b)
    az = None if a_zero_point is None else _host(a_zero_point)
    bz = None if b_zero_point is None else _host(b_zero_point)
    y = out if out is not None else _like(a, _mm_shape(a, b), np.int32)
    with _OMT(y) as hy, _OMT(a) as ha, _OMT(b) as hb, _OMT(az) as haz, _OMT(bz) as hbz:
        _lib.om_mi355x_MatMulInteger(hy, ha, hb, haz, hbz)
    _check()
    return y


def MatMulIntegerDequant(a: Tensor, b: Tensor, a_zero_point: Optional[Tensor],
                         b_zero_point: Optional[Tensor], a_scale: Tensor, b_scale: Tensor,
                         bias: Optional[Tensor] = None, out: Optional[Tensor] = None,
                         activation: int = ACTIVATION_NONE) -> Tensor:
    load()
    a, b = _host(a), _host(b)
    a_scale, b_scale = _host(a_scale, np.float32), _host(b_scale, np.float32)
    az = None if a_zero_point is None else _host(a_zero_point)
    bz = None if b_zero_point is None else _host(b_zero_point)
    bias = None if bias is None else _host(bias, np.float32)
    y = out if out is not None else _like(a, _mm_shape(a, b), np.float32)
    with _OMT(y) as hy, _OMT(a) as ha, _OMT(b) as hb, _OMT(az) as haz, _OMT(bz) as hbz, \
            _OMT(a_scale) as has, _OMT(b_scale) as hbs, _OMT(bias) as hbias:
        _lib.om_mi355x_MatMulIntegerDequant(hy, ha, hb, haz, hbz, has, hbs, hbias, int(activation))
    _check()
    return y


def QLinearMatMul(a: Tensor, a_scale: Tensor, a_zero_point: Tensor, b: Tensor,
                  b_scale: Tensor, b_zero_point: Tensor, y_scale: Tensor,
                  y_zero_point: Tensor, narrow_mode: int = WRAP,
                  out: Optional[Tensor] = None) -> Tensor:
    load()
    a, b = _host(a), _host(b)
    a_scale, b_scale = _host(a_scale, np.float32), _host(b_scale, np.float32)
    y_scale = _host(y_scale, np.float32)
    az, bz, yz = _host(a_zero_point), _host(b_zero_point), _host(y_zero_point)
    y = out if out is not None else _like(a, _mm_shape(a, b), yz.dtype)
    with _OMT(y) as hy, _OMT(a) as ha, _OMT(a_scale) as has, _OMT(az) as haz, \
            _OMT(b) as hb, _OMT(b_scale) as hbs, _OMT(bz) as hbz, \
            _OMT(y_scale) as hys, _OMT(yz) as hyz:
        _lib.om_mi355x_QLinearMatMul(hy, ha, has, haz, hb, hbs, hbz, hys, hyz, narrow_mode)
    _check()
    return y


def DynQuantMatMulDequant(x: Tensor, b: Tensor, b_zero_point: Optional[Tensor],
                          b_scale: Tensor, bias: Optional[Tensor] = None,
                          out: Optional[Tensor] = None, activation: int = ACTIVATION_NONE) -> Tensor:
    load()
    x, b, b_scale = _host(x), _host(b), _host(b_scale, np.float32)
    bz = None if b_zero_point is None else _host(b_zero_point)
    bias = None if bias is None else _host(bias, np.float32)
    y = out if out is not None else _like(x, _mm_shape(x, b), np.float32)
    with _OMT(y) as hy, _OMT(x) as hx, _OMT(b) as hb, _OMT(bz) as hbz, _OMT(b_scale) as hbs, \
            _OMT(bias) as hbias:
        _emit_quant_mode()
        _lib.om_mi355x_DynQuantMatMulDequant(hy, hx, hb, hbz, hbs, hbias, int(activation))
    _check()
    return y


def DynQuantMatMulDequantLimits(x: Tensor, b: Tensor, b_zero_point: Optional[Tensor],
                                b_scale: Tensor, bias: Optional[Tensor] = None,
                                out: Optional[Tensor] = None, activation: int = ACTIVATION_NONE,
                                x_limits: Optional[Tensor] = None, y_limits: Optional[Tensor] = None,
                                want_limits: bool = True):
    """om_mi355x_DynQuantMatMulDequantLimits: returns (y, y_limits); y_limits is
    None when want_limits is false and none were passed in."""
    load()
    x, b, b_scale = _host(x), _host(b), _host(b_scale, np.float32)
    bz = None if b_zero_point is None else _host(b_zero_point)
    bias = None if bias is None else _host(bias, np.float32)
    xl = None if x_limits is None else _host(x_limits, np.float32)
    y = out if out is not None else _like(x, _mm_shape(x, b), np.float32)
    yl = y_limits
    if yl is None and want_limits:
        yl = _like(x, (2,), np.float32)
    with _OMT(y) as hy, _OMT(yl) as hyl, _OMT(x) as hx, _OMT(xl) as hxl, _OMT(b) as hb, \
            _OMT(bz) as hbz, _OMT(b_scale) as hbs, _OMT(bias) as hbias:
        _emit_quant_mode()
        _lib.om_mi355x_DynQuantMatMulDequantLimits(hy, hyl, hx, hxl, hb, hbz, hbs, hbias, int(activation))
    _check()
    return y, yl


class PreparedCall:
    """An entry point bound once to fixed operands: the OMTensor wrappers are
    built a single time, so that calling it costs one C call (what a compiled
    model pays), not a Python marshalling pass.  ``operands`` follow the C
    signature: tensors (or None) first, then integer attributes."""

    def __init__(self, entry: str, *operands):
        load()
        self._fn = getattr(_lib, entry)
        self._wrappers = []
        self._args = []
        for o in operands:
            if isinstance(o, (int, np.integer)) and not isinstance(o, np.ndarray):
                self._args.append(int(o))
            else:
                w = _OMT(o)
                self._wrappers.append(w)
                self._args.append(w.handle)

    def __call__(self):
        self._fn(*self._args)

    def check(self):
        _check()

    def close(self):
        for w in self._wrappers:
            w.__exit__()
        self._wrappers = []
