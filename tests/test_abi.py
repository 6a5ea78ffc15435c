"""Boundary checks that need no GPU: the C-ABI library loads and exports every
symbol the headers declare, the OMTensor layout is the reference's, arguments
are validated, and without a device the entry points fail loudly (there is no
CPU path behind them)."""
import ctypes
import errno
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
REF_RUNTIME = os.path.join(ROOT, "oracle", "_ref", "libomruntime_ref.so")


def _declared(header, pattern):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(pattern, text)))


def test_library_exports_every_declared_symbol(rt):
    lib = rt.load()
    names = _declared("om_mi355x.h", r"\b(om_mi355x_\w+|OM\w+AccelMI355X)\s*\(")
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), f"{n} declared in om_mi355x.h but not exported"
    assert ctypes.c_long.in_dll(lib, "OMIsInitAccelMI355X") is not None
    shim = ctypes.CDLL(rt.SHIM_PATH)
    for n in _declared("om_tensor_abi.h", r"\b(omTensor\w+)\s*\("):
        assert hasattr(shim, n), f"{n} declared in om_tensor_abi.h but not exported"


def test_runtime_library_does_not_define_tensor_accessors(rt):
    # A compiled model brings the omTensor* symbols from libcruntime; the runtime
    # library must only reference them, or the model link would see duplicates.
    import subprocess
    out = subprocess.check_output(["nm", "-D", "--defined-only", rt.LIB_PATH], text=True)
    assert "omTensorGetDataPtr" not in out
    und = subprocess.check_output(["nm", "-D", "--undefined-only", rt.LIB_PATH], text=True)
    assert "omTensorGetDataPtr" in und


def test_runtime_does_not_depend_on_the_test_shim(rt):
    """Neither form of the runtime names libom_tensor_shim.so: the omTensor*
    accessors are resolved by whatever provides them in the process (a
    compiled model's libcruntime; the shim in these tests)."""
    import subprocess
    dyn = subprocess.check_output(["readelf", "-d", rt.LIB_PATH], text=True)
    needed = re.findall(r"\(NEEDED\).*\[(.*?)\]", dyn)
    assert needed and not any("tensor_shim" in n for n in needed), needed
    assert any(n.startswith("libamdhip64") for n in needed)


def test_static_archive_links_into_a_model_library(rt, tmp_path):
    """libRuntimeMI355X.a is what a compiled model links against, as the
    reference's accelerators package their runtimes
    (src/Accelerators/NNPA/Runtime/CMakeLists.txt:5-35; added to the link line
    by CCM_SHARED_LIB_DEPS, src/Accelerators/NNPA/NNPAAccelerator.cpp:60-81).
    A stand-in for a model -- one C function that references every entry point
    of include/om_mi355x.h -- is linked into a shared library against the
    archive and libamdhip64 the way src/Compiler/CompilerUtils.cpp links
    models (C++ driver, -shared, -l<dep> after the object), loaded beside an
    OMTensor provider, and called: the version handshake answers."""
    import subprocess
    archive = os.path.join(os.path.dirname(rt.LIB_PATH), "libRuntimeMI355X.a")
    assert os.path.exists(archive), "libRuntimeMI355X.a is not built"
    names = _declared("om_mi355x.h", r"\b(om_mi355x_\w+|OM\w+AccelMI355X)\s*\(")
    stub = tmp_path / "model_stub.c"
    stub.write_text(
        '#include "om_mi355x.h"\n'
        "const void *model_entry_points[] = {\n"
        + "".join(f"  (const void *){n},\n" for n in names)
        + "};\nunsigned long long model_handshake(unsigned long long v) {\n"
          "  return OMInitCompatibleAccelMI355X(v);\n}\n")
    obj, lib = tmp_path / "model_stub.o", tmp_path / "model.so"
    subprocess.check_call(["gcc", "-c", "-fPIC", "-I", INCLUDE, str(stub), "-o", str(obj)])
    subprocess.check_call(["g++", "-shared", "-fPIC", str(obj), "-o", str(lib),
                           "-L", os.path.dirname(archive), "-lRuntimeMI355X",
                           "-L", "/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"])
    defined = subprocess.check_output(["nm", "-D", "--defined-only", str(lib)], text=True)
    assert "om_mi355x_QLinearMatMul" in defined and "omTensorGetDataPtr" not in defined
    ctypes.CDLL(rt.SHIM_PATH, mode=ctypes.RTLD_GLOBAL)
    model = ctypes.CDLL(str(lib))
    model.model_handshake.restype = ctypes.c_uint64
    model.model_handshake.argtypes = [ctypes.c_uint64]
    # another major version is refused with or without a GPU
    assert model.model_handshake(0x00FF0000) == 0
    if not _no_gpu():
        assert model.model_handshake(rt.VERSION) == 1


@pytest.mark.skipif(not os.path.exists(REF_RUNTIME), reason="oracle/_ref not built (no reference tree)")
def test_omtensor_layout_matches_reference_runtime(rt):
    """A tensor built by the reference's own C runtime is read correctly by our
    accessors and vice versa (struct of src/Runtime/OMTensor.inc:125-140)."""
    ref = ctypes.CDLL(REF_RUNTIME)
    shim = ctypes.CDLL(rt.SHIM_PATH)
    P, I64 = ctypes.c_void_p, ctypes.c_int64
    for lib in (ref, shim):
        lib.omTensorCreate.restype = P
        lib.omTensorCreate.argtypes = [P, ctypes.POINTER(I64), I64, ctypes.c_int]
        lib.omTensorDestroy.argtypes = [P]
        lib.omTensorGetDataPtr.restype = P
        lib.omTensorGetDataPtr.argtypes = [P]
        lib.omTensorGetShape.restype = ctypes.POINTER(I64)
        lib.omTensorGetShape.argtypes = [P]
        lib.omTensorGetStrides.restype = ctypes.POINTER(I64)
        lib.omTensorGetStrides.argtypes = [P]
        lib.omTensorGetRank.restype = I64
        lib.omTensorGetRank.argtypes = [P]
        lib.omTensorGetDataType.restype = ctypes.c_int
        lib.omTensorGetDataType.argtypes = [P]
        lib.omTensorGetNumElems.restype = I64
        lib.omTensorGetNumElems.argtypes = [P]
        lib.omTensorGetBufferSize.restype = I64
        lib.omTensorGetBufferSize.argtypes = [P]
    data = np.arange(2 * 3 * 5, dtype=np.int32)
    shape = (I64 * 3)(2, 3, 5)
    for maker, reader in ((ref, shim), (shim, ref)):
        for dtype_code, itemsize in ((6, 4), (1, 4), (2, 1), (3, 1)):
            t = maker.omTensorCreate(data.ctypes.data, shape, 3, dtype_code)
            assert reader.omTensorGetDataPtr(t) == data.ctypes.data
            assert reader.omTensorGetRank(t) == 3
            assert [reader.omTensorGetShape(t)[i] for i in range(3)] == [2, 3, 5]
            assert [reader.omTensorGetStrides(t)[i] for i in range(3)] == [15, 5, 1]
            assert reader.omTensorGetDataType(t) == dtype_code
            assert reader.omTensorGetNumElems(t) == 30
            assert reader.omTensorGetBufferSize(t) == 30 * itemsize
            maker.omTensorDestroy(t)
    # rank 0 (scalars such as y_scale)
    t = ref.omTensorCreate(data.ctypes.data, shape, 0, 1)
    assert shim.omTensorGetRank(t) == 0 and shim.omTensorGetNumElems(t) == 1
    ref.omTensorDestroy(t)


def _no_gpu():
    return not os.path.exists("/dev/kfd")


def test_argument_validation_sets_einval(rt):
    x = np.zeros((4, 6), np.float32)
    with pytest.raises(rt.RuntimeError_, match="scale has 5 entries"):
        rt.QuantizeLinear(x, np.ones(5, np.float32), np.zeros(5, np.uint8), axis=1)
    assert ctypes.get_errno() in (0, errno.EINVAL)
    with pytest.raises(rt.RuntimeError_, match="zero point"):
        rt.QuantizeLinear(x, np.ones(6, np.float32), np.zeros(3, np.uint8), axis=1)
    with pytest.raises(rt.RuntimeError_, match="inner dimensions differ"):
        rt.MatMulInteger(np.zeros((4, 6), np.uint8), np.zeros((5, 3), np.int8))
    with pytest.raises(rt.RuntimeError_, match="zero point's type"):
        rt.MatMulInteger(np.zeros((4, 6), np.uint8), np.zeros((6, 3), np.int8),
                         np.zeros((), np.int8), None)
    with pytest.raises(rt.RuntimeError_, match="expected 1 or 3"):
        rt.MatMulInteger(np.zeros((4, 6), np.uint8), np.zeros((6, 3), np.int8),
                         None, np.zeros(2, np.int8))
    with pytest.raises(rt.RuntimeError_, match="expected f32 x"):
        rt.DynamicQuantizeLinear(np.zeros(4, np.int32))
    with pytest.raises(rt.RuntimeError_, match="bias must be f32, scalar or"):
        rt.MatMulIntegerDequant(np.zeros((4, 6), np.uint8), np.zeros((6, 3), np.int8), None, None,
                                np.float32(1), np.float32(1), np.zeros(2, np.float32))
    # a dimension that was never resolved
    buf = np.zeros(16, np.float32)
    shape = (ctypes.c_int64 * 2)(-1, 4)
    h = rt._shim.omTensorCreate(buf.ctypes.data, shape, 2, 1)
    try:
        rt._lib.om_mi355x_DynamicQuantizeLinear(h, h, h, h)
        with pytest.raises(rt.RuntimeError_, match="dimension 0 is -1"):
            rt._check()
    finally:
        rt._shim.omTensorDestroy(h)


def test_incompatible_version_is_refused(rt):
    lib = rt.load()
    assert lib.OMInitCompatibleAccelMI355X(0x00020000) == 0   # newer major
    assert lib.OMInitCompatibleAccelMI355X(0x00000100) == 0   # older major: signatures have changed since
    assert lib.OMInitCompatibleAccelMI355X(0x00010100) == 0   # newer minor
    rt._lib.om_mi355x_last_error()


@pytest.mark.skipif(not _no_gpu(), reason="only meaningful on a box without a GPU")
def test_without_a_gpu_the_ops_fail_loudly(rt):
    lib = rt.load()
    assert lib.OMInitCompatibleAccelMI355X(rt.VERSION) == 0    # run_main_graph would return NULL
    with pytest.raises(rt.RuntimeError_, match="accelerator unavailable"):
        rt.QuantizeLinear(np.ones(8, np.float32), np.float32(0.5), np.array(3, np.uint8))
    with pytest.raises(rt.RuntimeError_, match="accelerator unavailable"):
        rt.MatMulInteger(np.ones((2, 2), np.uint8), np.ones((2, 2), np.int8))


PLUGIN = os.path.join(ROOT, "onnx-mlir_amd", "accelerator")


def _plugin_sources():
    out = []
    for base, _, files in os.walk(os.path.join(PLUGIN, "src")):
        out += [os.path.join(base, f) for f in files if f.endswith((".cpp", ".hpp"))]
    return out


def test_compiler_plugin_calls_only_exported_symbols(rt):
    """Every callee the onnx-mlir plug-in emits a krnl.call to is a symbol of the
    runtime, with as many parameters as the plug-in passes."""
    lib = rt.load()
    header = open(os.path.join(INCLUDE, "om_mi355x.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    callees = set()
    for path in _plugin_sources():
        callees |= set(re.findall(r'"(om_mi355x_\w+)"', open(path).read()))
    assert {"om_mi355x_QuantizeLinear", "om_mi355x_DequantizeLinear",
            "om_mi355x_DynamicQuantizeLinear", "om_mi355x_MatMulInteger",
            "om_mi355x_QLinearMatMul", "om_mi355x_MatMulIntegerDequant",
            "om_mi355x_DynQuantMatMulDequant", "om_mi355x_MarkConstant",
            "om_mi355x_KeepOnDevice", "om_mi355x_Release", "om_mi355x_SetQuantMode"} <= callees
    for name in callees:
        assert hasattr(lib, name), f"plug-in calls {name}, which the runtime lacks"
    # parameter counts: results + operands + integer attributes of each pattern
    passed = {"om_mi355x_QuantizeLinear": 1 + 3 + 2, "om_mi355x_DequantizeLinear": 1 + 3 + 1,
              "om_mi355x_DynamicQuantizeLinear": 3 + 1, "om_mi355x_MatMulInteger": 1 + 4,
              "om_mi355x_QLinearMatMul": 1 + 8 + 1, "om_mi355x_MatMulIntegerDequant": 1 + 7 + 1,
              "om_mi355x_DynQuantMatMulDequant": 1 + 5 + 1, "om_mi355x_MarkConstant": 1,
              "om_mi355x_KeepOnDevice": 1, "om_mi355x_Release": 1,
              "om_mi355x_SetQuantMode": 1 + 1}   # the anchor buffer + `mode`
    for name, count in passed.items():
        m = re.search(r"\b%s\s*\(([^)]*)\)" % name, header)
        assert m, name
        assert len([p for p in m.group(1).split(",") if p.strip()]) == count, name


def test_quant_mode_constants_agree_everywhere():
    """The two bits of om_mi355x_SetQuantMode are spelled in the header, the
    Python mirror, the oracle and (as literals) the plug-in: same values."""
    import om_mi355x
    import oracle_lib
    header = open(os.path.join(INCLUDE, "om_mi355x.h")).read()
    recip = int(re.search(r"#define\s+OM_MI355X_QUANT_RECIPROCAL\s+(\d+)", header).group(1))
    no_zp = int(re.search(r"#define\s+OM_MI355X_QUANT_NO_ZERO_POINT\s+(\d+)", header).group(1))
    assert (recip, no_zp) == (1, 2)
    assert (om_mi355x.QUANT_RECIPROCAL, om_mi355x.QUANT_NO_ZERO_POINT) == (recip, no_zp)
    assert (oracle_lib.RECIPROCAL, oracle_lib.NO_ZERO_POINT) == (recip, no_zp)
    oracle_h = open(os.path.join(ROOT, "oracle", "om_oracle.h")).read()
    assert re.search(r"OM_ORACLE_RECIPROCAL\s*=\s*1\s*,\s*OM_ORACLE_NO_ZERO_POINT\s*=\s*2", oracle_h)
    conv = open(os.path.join(PLUGIN, "src", "Accelerators", "MI355X", "Conversion", "ONNXToMI355XCall.cpp")).read()
    assert "mode |= 1; // OM_MI355X_QUANT_RECIPROCAL" in conv and "mode |= 2; // OM_MI355X_QUANT_NO_ZERO_POINT" in conv


def test_compiler_plugin_version_matches_runtime():
    header = open(os.path.join(INCLUDE, "om_mi355x.h")).read()
    runtime = int(re.search(r"#define\s+OM_MI355X_VERSION\s+(0x[0-9a-fA-F]+)", header).group(1), 16)
    accel = open(os.path.join(PLUGIN, "src", "Accelerators", "MI355X", "MI355XAccelerator.cpp")).read()
    plugin = int(re.search(r"kRuntimeVersion\s*=\s*(0x[0-9a-fA-F]+)", accel).group(1), 16)
    assert plugin == runtime


def test_compiler_plugin_lit_tests_name_real_entry_points(rt):
    lib = rt.load()
    lit = os.path.join(PLUGIN, "test", "mlir", "accelerators", "mi355x")
    files = [f for f in os.listdir(lit) if f.endswith(".mlir")]
    assert len(files) >= 5
    for f in files:
        text = open(os.path.join(lit, f)).read()
        assert "// RUN: onnx-mlir-opt --maccel=MI355X" in text
        for name in set(re.findall(r'"(om_mi355x_\w+)"', text)):
            assert hasattr(lib, name), (f, name)


def test_benchmark_model_texts_are_what_their_generator_writes():
    """bench/models/*.mlir are the five configurations as ONNX-dialect text for
    the reference compiler; they must stay in step with the script beside them,
    and their shapes with the workloads the GPU bench runs."""
    import importlib.util
    models = os.path.join(ROOT, "bench", "models")
    spec = importlib.util.spec_from_file_location("make_models", os.path.join(models, "make_models.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for n in range(1, 6):
        assert f"cfg{n}.mlir" in mod.MODELS
    for name, text in mod.MODELS.items():
        with open(os.path.join(models, name)) as fh:
            assert fh.read() == text, name
        assert text.count("{") == text.count("}") and '"onnx.EntryPoint"() {func = @main_graph}' in text
    assert "tensor<4096x768xui8>" in mod.MODELS["cfg4_matmulinteger.mlir"]
    assert "tensor<768x3072xi8>" in mod.MODELS["cfg4_matmulinteger.mlir"]
    assert "tensor<8191x32767xf32>" in mod.MODELS["cfg2_per_axis_ragged.mlir"]


def test_reference_compiler_leg_of_the_bench_is_skipped_without_the_compiler(monkeypatch):
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_main", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    monkeypatch.setenv("PATH", "/nonexistent")
    assert bench.onnx_mlir_leg(None, None, None, None, None, None) is None


def test_python_module_version_is_the_headers():
    import om_mi355x
    header = open(os.path.join(INCLUDE, "om_mi355x.h")).read()
    assert om_mi355x.VERSION == int(re.search(r"#define\s+OM_MI355X_VERSION\s+(0x[0-9a-fA-F]+)", header).group(1), 16)
