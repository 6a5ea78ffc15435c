// RUN: onnx-mlir-opt --maccel=MI355X --mi355x-fuse-gelu --shape-inference --fuse-quantized-matmul-for-mi355x --canonicalize %s -split-input-file | FileCheck %s
// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --fuse-quantized-matmul-for-mi355x --canonicalize %s -split-input-file | FileCheck --check-prefix=DEFAULT %s

// With --mi355x-fuse-gelu an exact Gelu on the biased result becomes
// `activation` = 2 of the same call; without the option it stays an op of its
// own behind the call, because the two sides evaluate erf differently.
func.func @whole_layer_with_bias_and_gelu(%x: tensor<128x768xf32>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>, %bias: tensor<3072xf32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x3072xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  %z = "onnx.Add"(%y, %bias) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %r = "onnx.Gelu"(%z) {approximate = "none"} : (tensor<*xf32>) -> tensor<*xf32>
  return %r : tensor<*xf32>
// CHECK-LABEL:  func.func @whole_layer_with_bias_and_gelu
// CHECK-SAME:   ([[X:%.+]]: tensor<128x768xf32>, [[W:%.+]]: tensor<768x3072xi8>, [[WS:%.+]]: tensor<3072xf32>, [[BIAS:%.+]]: tensor<3072xf32>)
// CHECK:        [[R:%.+]] = "onnx.Custom"([[X]], [[W]], {{%.+}}, [[WS]], [[BIAS]])
// CHECK-SAME:   activation = 2 : i64
// CHECK-SAME:   function_name = "om_mi355x_DynQuantMatMulDequant"
// CHECK-NOT:    onnx.Gelu
// CHECK:        return [[R]]
// DEFAULT-LABEL: func.func @whole_layer_with_bias_and_gelu
// DEFAULT:       [[C:%.+]] = "onnx.Custom"
// DEFAULT-SAME:  activation = 0 : i64
// DEFAULT:       [[R:%.+]] = "onnx.Gelu"([[C]])
// DEFAULT:       return [[R]]
}

// -----

// The tanh form of Gelu is another function: it is never taken into the call.
func.func @tanh_gelu_stays(%x: tensor<128x768xf32>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x3072xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  %r = "onnx.Gelu"(%y) {approximate = "tanh"} : (tensor<*xf32>) -> tensor<*xf32>
  return %r : tensor<*xf32>
// CHECK-LABEL:  func.func @tanh_gelu_stays
// CHECK:        [[C:%.+]] = "onnx.Custom"
// CHECK-SAME:   activation = 0 : i64
// CHECK:        [[R:%.+]] = "onnx.Gelu"([[C]])
// CHECK:        return [[R]]
}
