// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --fuse-quantized-matmul-for-mi355x --canonicalize %s -split-input-file | FileCheck %s

// The five-op chain of a dynamically quantised linear layer becomes one op.
func.func @whole_layer(%x: tensor<128x768xf32>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>) -> tensor<*xf32> {
  %wzp = onnx.Constant dense<0> : tensor<i8>
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %wzp) : (tensor<*xui8>, tensor<768x3072xi8>, tensor<*xui8>, tensor<i8>) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @whole_layer
// CHECK-SAME:   ([[X:%.+]]: tensor<128x768xf32>, [[W:%.+]]: tensor<768x3072xi8>, [[WS:%.+]]: tensor<3072xf32>)
// CHECK:        [[WZP:%.+]] = onnx.Constant dense<0> : tensor<i8>
// CHECK:        [[NONE:%.+]] = "onnx.NoValue"
// CHECK:        [[Y:%.+]] = "onnx.Custom"([[X]], [[W]], [[WZP]], [[WS]], [[NONE]])
// CHECK-SAME:   function_name = "om_mi355x_DynQuantMatMulDequant"
// CHECK-SAME:   -> tensor<128x3072xf32>
// CHECK-NOT:    onnx.DynamicQuantizeLinear
// CHECK-NOT:    onnx.MatMulInteger
// CHECK-NOT:    onnx.Mul
// CHECK:        return [[Y]]
}

// -----

// The quantised activation has a second user: it must stay, and only the
// matmul and its scaling are fused.
func.func @activation_reused(%x: tensor<128x768xf32>, %w: tensor<768x768xi8>, %ws: tensor<f32>) -> (tensor<*xf32>, tensor<*xui8>) {
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x768xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<f32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%s, %f) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %y, %aq : tensor<*xf32>, tensor<*xui8>
// CHECK-LABEL:  func.func @activation_reused
// CHECK:        [[AQ:%.+]], [[AS:%.+]], [[AZP:%.+]] = "onnx.DynamicQuantizeLinear"
// CHECK:        [[Y:%.+]] = "onnx.Custom"([[AQ]], {{%.+}}, [[AZP]], {{%.+}}, [[AS]], {{%.+}}, {{%.+}})
// CHECK-SAME:   function_name = "om_mi355x_MatMulIntegerDequant"
// CHECK-NOT:    onnx.MatMulInteger
// CHECK:        return [[Y]], [[AQ]]
}

// -----

// The bias of the layer is added to the scaled result and nothing else uses
// that result: the Add goes into the same call.
func.func @whole_layer_with_bias(%x: tensor<128x768xf32>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>, %bias: tensor<3072xf32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x3072xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  %z = "onnx.Add"(%bias, %y) : (tensor<3072xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %z : tensor<*xf32>
// CHECK-LABEL:  func.func @whole_layer_with_bias
// CHECK-SAME:   ([[X:%.+]]: tensor<128x768xf32>, [[W:%.+]]: tensor<768x3072xi8>, [[WS:%.+]]: tensor<3072xf32>, [[BIAS:%.+]]: tensor<3072xf32>)
// CHECK:        [[Z:%.+]] = "onnx.Custom"([[X]], [[W]], {{%.+}}, [[WS]], [[BIAS]])
// CHECK-SAME:   function_name = "om_mi355x_DynQuantMatMulDequant"
// CHECK-SAME:   -> tensor<128x3072xf32>
// CHECK-NOT:    onnx.Add
// CHECK-NOT:    onnx.Mul
// CHECK:        return [[Z]]
}

// -----

// A second user of the scaled result keeps the Add outside the call.
func.func @bias_not_taken(%a: tensor<8x16xui8>, %w: tensor<16x4xi8>, %azp: tensor<ui8>, %as: tensor<f32>, %ws: tensor<f32>, %bias: tensor<4xf32>) -> (tensor<*xf32>, tensor<*xf32>) {
  %none = "onnx.NoValue"() {value} : () -> none
  %acc = "onnx.MatMulInteger"(%a, %w, %azp, %none) : (tensor<8x16xui8>, tensor<16x4xi8>, tensor<ui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<f32>, tensor<f32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  %z = "onnx.Add"(%y, %bias) : (tensor<*xf32>, tensor<4xf32>) -> tensor<*xf32>
  return %z, %y : tensor<*xf32>, tensor<*xf32>
// CHECK-LABEL:  func.func @bias_not_taken
// CHECK:        [[Y:%.+]] = "onnx.Custom"({{.*}})
// CHECK-SAME:   function_name = "om_mi355x_MatMulIntegerDequant"
// CHECK:        [[Z:%.+]] = "onnx.Add"([[Y]], {{%.+}})
// CHECK:        return [[Z]], [[Y]]
}

// -----

// (f32(acc) * a_scale) * b_scale rounds differently from what the fused entry
// point computes: not fused.
func.func @other_association(%a: tensor<8x16xui8>, %w: tensor<16x4xi8>, %azp: tensor<ui8>, %as: tensor<f32>, %ws: tensor<f32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %acc = "onnx.MatMulInteger"(%a, %w, %azp, %none) : (tensor<8x16xui8>, tensor<16x4xi8>, tensor<ui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %t = "onnx.Mul"(%f, %as) : (tensor<*xf32>, tensor<f32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%t, %ws) : (tensor<*xf32>, tensor<f32>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @other_association
// CHECK-NOT:    onnx.Custom
// CHECK:        onnx.MatMulInteger
}

// -----

// A batched right-hand side is not a linear layer's weight matrix: the chain
// is left as it is (the fused entry points take a 2-D B).
func.func @batched_rhs_is_left_alone(%a: tensor<4x128x64xui8>, %b: tensor<4x64x32xi8>, %azp: tensor<ui8>, %as: tensor<f32>, %bs: tensor<32xf32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %acc = "onnx.MatMulInteger"(%a, %b, %azp, %none) : (tensor<4x128x64xui8>, tensor<4x64x32xi8>, tensor<ui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %bs) : (tensor<f32>, tensor<32xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @batched_rhs_is_left_alone
// CHECK:        "onnx.MatMulInteger"
// CHECK:        "onnx.Cast"
// CHECK:        "onnx.Mul"
// CHECK-NOT:    onnx.Custom
}

// -----

// A Relu on the biased result, with no other user in between, becomes the
// `activation` attribute of the same call.
func.func @whole_layer_with_bias_and_relu(%x: tensor<128x768xf32>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>, %bias: tensor<3072xf32>) -> tensor<*xf32> {
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x3072xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  %z = "onnx.Add"(%y, %bias) : (tensor<*xf32>, tensor<3072xf32>) -> tensor<*xf32>
  %r = "onnx.Relu"(%z) : (tensor<*xf32>) -> tensor<*xf32>
  return %r : tensor<*xf32>
// CHECK-LABEL:  func.func @whole_layer_with_bias_and_relu
// CHECK-SAME:   ([[X:%.+]]: tensor<128x768xf32>, [[W:%.+]]: tensor<768x3072xi8>, [[WS:%.+]]: tensor<3072xf32>, [[BIAS:%.+]]: tensor<3072xf32>)
// CHECK:        [[R:%.+]] = "onnx.Custom"([[X]], [[W]], {{%.+}}, [[WS]], [[BIAS]])
// CHECK-SAME:   activation = 1 : i64
// CHECK-SAME:   function_name = "om_mi355x_DynQuantMatMulDequant"
// CHECK-NOT:    onnx.Relu
// CHECK-NOT:    onnx.Add
// CHECK:        return [[R]]
}
