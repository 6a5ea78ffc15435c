// RUN: onnx-mlir-opt --maccel=MI355X --mi355x-qlinear-narrow=saturate --shape-inference --convert-onnx-to-krnl %s | FileCheck %s

func.func @qlinear_matmul(%a: tensor<2x4xi8>, %as: tensor<f32>, %azp: tensor<i8>, %b: tensor<4x3xi8>, %bs: tensor<f32>, %bzp: tensor<i8>, %ys: tensor<f32>, %yzp: tensor<i8>) -> tensor<*xi8> {
  %y = "onnx.QLinearMatMul"(%a, %as, %azp, %b, %bs, %bzp, %ys, %yzp) : (tensor<2x4xi8>, tensor<f32>, tensor<i8>, tensor<4x3xi8>, tensor<f32>, tensor<i8>, tensor<f32>, tensor<i8>) -> tensor<*xi8>
  return %y : tensor<*xi8>
// CHECK-LABEL:  func.func @qlinear_matmul
// CHECK:        funcName = "om_mi355x_QLinearMatMul"
// CHECK-SAME:   narrow_mode = 1 : i64
}
