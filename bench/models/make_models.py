#!/usr/bin/env python3
"""Writes the five benchmark configurations as ONNX-dialect MLIR text, the
form `onnx-mlir` takes directly (src/Compiler/CompilerUtils.cpp:694,729-730), so
that the reference compiler -- where one is installed -- can build the CPU
model of each configuration without the `onnx` Python package:

    onnx-mlir -O3 --parallel cfg4.mlir -o cfg4     # -> cfg4.so, run_main_graph

Weights are graph inputs, which keeps the files small (the reference folds
MatMulInteger only when both operands are constants,
src/Dialect/ONNX/Transforms/ConstProp.td:997-1003).  Per-axis QuantizeLinear /
DequantizeLinear are written decomposed into Div/Round/Add/Clip/Cast and
Cast/Sub/Mul, the form the reference's CPU lowering can compile: its own
lowerings take per-tensor scales only
(src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:40-47), while
onnx.Round is the same round-half-to-even
(src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:1394-1403) and onnx.Clip the
same max-then-min (:1414-1426).

Run from this directory:  python make_models.py
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def t(shape, ty):
    return "tensor<" + "x".join([str(d) for d in shape] + [ty]) + ">"


def entry():
    return '  "onnx.EntryPoint"() {func = @main_graph} : () -> ()\n'


def dyn_linear(M, K, N, per_column, b_scale=None):
    """DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul (configs 1, 4, 5)."""
    x, b, xq, acc, y = t((M, K), "f32"), t((K, N), "i8"), t((M, K), "ui8"), t((M, N), "i32"), t((M, N), "f32")
    f, u8, i8 = "tensor<f32>", "tensor<ui8>", "tensor<i8>"
    if per_column:
        bs = t((N,), "f32")
        sig = f"%X: {x}, %B: {b}, %bs: {bs}"
        scale = ""
    else:
        bs = f
        sig = f"%X: {x}, %B: {b}"
        scale = f"    %bs = onnx.Constant dense<{b_scale:e}> : {f}\n"
    return (
        "module {\n"
        f"  func.func @main_graph({sig}) -> {y} {{\n"
        f"    %bzp = onnx.Constant dense<0> : {i8}\n"
        f"{scale}"
        f'    %xq, %xs, %xzp = "onnx.DynamicQuantizeLinear"(%X) : ({x}) -> ({xq}, {f}, {u8})\n'
        f'    %acc = "onnx.MatMulInteger"(%xq, %B, %xzp, %bzp) : ({xq}, {b}, {u8}, {i8}) -> {acc}\n'
        f'    %c = "onnx.Cast"(%acc) {{to = f32}} : ({acc}) -> {y}\n'
        f'    %s = "onnx.Mul"(%xs, %bs) : ({f}, {bs}) -> {bs}\n'
        f'    %y = "onnx.Mul"(%c, %s) : ({y}, {bs}) -> {y}\n'
        f"    return %y : {y}\n"
        "  }\n" + entry() + "}\n")


def matmul_dequant(M, K, N):
    """MatMulInteger -> Cast -> Mul on already quantized activations: the op the
    headline number times."""
    a, b, acc, y = t((M, K), "ui8"), t((K, N), "i8"), t((M, N), "i32"), t((M, N), "f32")
    f, u8, bs = "tensor<f32>", "tensor<ui8>", t((N,), "f32")
    return (
        "module {\n"
        f"  func.func @main_graph(%A: {a}, %B: {b}, %azp: {u8}, %as: {f}, %bs: {bs}) -> {y} {{\n"
        '    %none = "onnx.NoValue"() {value} : () -> none\n'
        f'    %acc = "onnx.MatMulInteger"(%A, %B, %azp, %none) : ({a}, {b}, {u8}, none) -> {acc}\n'
        f'    %c = "onnx.Cast"(%acc) {{to = f32}} : ({acc}) -> {y}\n'
        f'    %s = "onnx.Mul"(%as, %bs) : ({f}, {bs}) -> {bs}\n'
        f'    %y = "onnx.Mul"(%c, %s) : ({y}, {bs}) -> {y}\n'
        f"    return %y : {y}\n"
        "  }\n" + entry() + "}\n")


def qdq_per_tensor(R, C):
    x, q = t((R, C), "f32"), t((R, C), "ui8")
    f, u8 = "tensor<f32>", "tensor<ui8>"
    return (
        "module {\n"
        f"  func.func @main_graph(%X: {x}, %s: {f}, %zp: {u8}) -> ({q}, {x}, {q}, {f}, {u8}) {{\n"
        f'    %q = "onnx.QuantizeLinear"(%X, %s, %zp) {{axis = 1 : si64}} : ({x}, {f}, {u8}) -> {q}\n'
        f'    %d = "onnx.DequantizeLinear"(%q, %s, %zp) {{axis = 1 : si64}} : ({q}, {f}, {u8}) -> {x}\n'
        f'    %dq, %ds, %dzp = "onnx.DynamicQuantizeLinear"(%X) : ({x}) -> ({q}, {f}, {u8})\n'
        f"    return %q, %d, %dq, %ds, %dzp : {q}, {x}, {q}, {f}, {u8}\n"
        "  }\n" + entry() + "}\n")


def qdq_per_axis(R, C):
    x, q = t((R, C), "f32"), t((R, C), "ui8")
    s, z, f = t((C,), "f32"), t((C,), "ui8"), "tensor<f32>"
    return (
        "module {\n"
        f"  func.func @main_graph(%X: {x}, %s: {s}, %zp: {z}) -> ({q}, {x}) {{\n"
        f"    %lo = onnx.Constant dense<0.000000e+00> : {f}\n"
        f"    %hi = onnx.Constant dense<2.550000e+02> : {f}\n"
        f'    %zf = "onnx.Cast"(%zp) {{to = f32}} : ({z}) -> {s}\n'
        f'    %v = "onnx.Div"(%X, %s) : ({x}, {s}) -> {x}\n'
        f'    %r = "onnx.Round"(%v) : ({x}) -> {x}\n'
        f'    %a = "onnx.Add"(%r, %zf) : ({x}, {s}) -> {x}\n'
        f'    %c = "onnx.Clip"(%a, %lo, %hi) : ({x}, {f}, {f}) -> {x}\n'
        f'    %q = "onnx.Cast"(%c) {{to = ui8}} : ({x}) -> {q}\n'
        f'    %qf = "onnx.Cast"(%q) {{to = f32}} : ({q}) -> {x}\n'
        f'    %m = "onnx.Sub"(%qf, %zf) : ({x}, {s}) -> {x}\n'
        f'    %d = "onnx.Mul"(%m, %s) : ({x}, {s}) -> {x}\n'
        f"    return %q, %d : {q}, {x}\n"
        "  }\n" + entry() + "}\n")


def qlinear(M, K, N):
    a, b, y = t((M, K), "ui8"), t((K, N), "ui8"), t((M, N), "ui8")
    f, u8 = "tensor<f32>", "tensor<ui8>"
    return (
        "module {\n"
        f"  func.func @main_graph(%A: {a}, %B: {b}) -> {y} {{\n"
        f"    %as = onnx.Constant dense<1.000000e-02> : {f}\n"
        f"    %azp = onnx.Constant dense<128> : {u8}\n"
        f"    %bs = onnx.Constant dense<5.000000e-03> : {f}\n"
        f"    %bzp = onnx.Constant dense<120> : {u8}\n"
        f"    %ys = onnx.Constant dense<5.000000e-01> : {f}\n"
        f"    %yzp = onnx.Constant dense<0> : {u8}\n"
        f'    %y = "onnx.QLinearMatMul"(%A, %as, %azp, %B, %bs, %bzp, %ys, %yzp) : '
        f"({a}, {f}, {u8}, {b}, {f}, {u8}, {f}, {u8}) -> {y}\n"
        f"    return %y : {y}\n"
        "  }\n" + entry() + "}\n")


MODELS = {
    "cfg1.mlir": dyn_linear(128, 768, 768, per_column=False, b_scale=0.02),
    "cfg2.mlir": qdq_per_tensor(8192, 32768),
    "cfg2_per_axis.mlir": qdq_per_axis(8192, 32768),
    "cfg2_per_axis_ragged.mlir": qdq_per_axis(8191, 32767),
    "cfg3.mlir": qlinear(512, 1024, 4096),
    "cfg4.mlir": dyn_linear(4096, 768, 3072, per_column=True),            # FFN-up
    "cfg4_qkv.mlir": dyn_linear(4096, 768, 2304, per_column=True),
    "cfg4_out.mlir": dyn_linear(4096, 768, 768, per_column=True),
    "cfg4_ffn_down.mlir": dyn_linear(4096, 3072, 768, per_column=True),
    "cfg4_matmulinteger.mlir": matmul_dequant(4096, 768, 3072),            # the headline op alone
    "cfg5.mlir": dyn_linear(2048, 4096, 11008, per_column=True),           # prefill up
    "cfg5_down.mlir": dyn_linear(2048, 11008, 4096, per_column=True),
    "cfg5_decode1.mlir": dyn_linear(1, 4096, 11008, per_column=True),
    "cfg5_decode4.mlir": dyn_linear(4, 4096, 11008, per_column=True),
    "cfg5_decode16.mlir": dyn_linear(16, 4096, 11008, per_column=True),
}

if __name__ == "__main__":
    for name, text in MODELS.items():
        with open(os.path.join(HERE, name), "w") as fh:
            fh.write(text)
        print("wrote", name)
