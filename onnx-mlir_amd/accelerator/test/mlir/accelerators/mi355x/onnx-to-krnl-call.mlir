// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --convert-onnx-to-krnl --canonicalize %s -split-input-file | FileCheck %s

// Results first, then the operands in ONNX order, then the integer attributes.
func.func @quantize_per_tensor(%x: tensor<4x768xf32>, %s: tensor<f32>, %zp: tensor<ui8>) -> tensor<*xui8> {
  %y = "onnx.QuantizeLinear"(%x, %s, %zp) {axis = 1 : si64, saturate = 1 : si64} : (tensor<4x768xf32>, tensor<f32>, tensor<ui8>) -> tensor<*xui8>
  return %y : tensor<*xui8>
// CHECK-LABEL:  func.func @quantize_per_tensor
// CHECK-SAME:   ([[X:%.+]]: memref<4x768xf32>, [[S:%.+]]: memref<f32>, [[ZP:%.+]]: memref<ui8>) -> memref<4x768xui8>
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<4x768xui8>
// CHECK:        "krnl.call"([[Y]], [[X]], [[S]], [[ZP]])
// CHECK-SAME:   funcName = "om_mi355x_QuantizeLinear", numOfOutput = 1 : si64
// CHECK-SAME:   axis = 1 : i64, saturate = 1 : i64
// CHECK-SAME:   (memref<4x768xui8>, memref<4x768xf32>, memref<f32>, memref<ui8>) -> ()
// CHECK-NOT:    krnl.iterate
// CHECK:        return [[Y]]
}

// -----

// An absent zero point stays in the operand list as `none` (NULL at run time).
func.func @quantize_no_zero_point(%x: tensor<?x768xf32>, %s: tensor<768xf32>) -> tensor<*xui8> {
  %none = "onnx.NoValue"() {value} : () -> none
  %y = "onnx.QuantizeLinear"(%x, %s, %none) {axis = 1 : si64} : (tensor<?x768xf32>, tensor<768xf32>, none) -> tensor<*xui8>
  return %y : tensor<*xui8>
// CHECK-LABEL:  func.func @quantize_no_zero_point
// CHECK:        [[DIM:%.+]] = memref.dim
// CHECK:        [[Y:%.+]] = memref.alloc([[DIM]]) {{.*}}: memref<?x768xui8>
// CHECK:        "krnl.call"([[Y]], {{%.+}}, {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_QuantizeLinear"
// CHECK-SAME:   (memref<?x768xui8>, memref<?x768xf32>, memref<768xf32>, none) -> ()
}

// -----

func.func @dequantize(%x: tensor<4x768xi8>, %s: tensor<f32>, %zp: tensor<i8>) -> tensor<*xf32> {
  %y = "onnx.DequantizeLinear"(%x, %s, %zp) {axis = 1 : si64} : (tensor<4x768xi8>, tensor<f32>, tensor<i8>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @dequantize
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<4x768xf32>
// CHECK:        "krnl.call"([[Y]], {{%.+}}, {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_DequantizeLinear", numOfOutput = 1 : si64
// CHECK-SAME:   axis = 1 : i64
}

// -----

// Three results, three leading parameters.
func.func @dynamic_quantize(%x: tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>) {
  %y, %s, %zp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  return %y, %s, %zp : tensor<*xui8>, tensor<*xf32>, tensor<*xui8>
// CHECK-LABEL:  func.func @dynamic_quantize
// CHECK-DAG:    [[Y:%.+]] = memref.alloc() {{.*}}: memref<128x768xui8>
// CHECK-DAG:    [[S:%.+]] = memref.alloc() {{.*}}: memref<f32>
// CHECK-DAG:    [[ZP:%.+]] = memref.alloc() {{.*}}: memref<ui8>
// CHECK:        "krnl.call"([[Y]], [[S]], [[ZP]], {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_DynamicQuantizeLinear", numOfOutput = 3 : si64
// CHECK:        return [[Y]], [[S]], [[ZP]]
}

// -----

// A constant right-hand side is announced to the runtime before its first use.
func.func @matmul_integer_constant_weight(%a: tensor<128x4xui8>, %azp: tensor<ui8>) -> tensor<*xi32> {
  %b = onnx.Constant dense<[[1, 2], [3, 4], [5, 6], [7, 8]]> : tensor<4x2xi8>
  %none = "onnx.NoValue"() {value} : () -> none
  %y = "onnx.MatMulInteger"(%a, %b, %azp, %none) : (tensor<128x4xui8>, tensor<4x2xi8>, tensor<ui8>, none) -> tensor<*xi32>
  return %y : tensor<*xi32>
// CHECK-LABEL:  func.func @matmul_integer_constant_weight
// CHECK:        [[B:%.+]] = "krnl.global"()
// CHECK:        "krnl.call"([[B]])
// CHECK-SAME:   funcName = "om_mi355x_MarkConstant", numOfOutput = 1 : si64
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<128x2xi32>
// CHECK:        "krnl.call"([[Y]], {{%.+}}, [[B]], {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_MatMulInteger", numOfOutput = 1 : si64
// CHECK-SAME:   (memref<128x2xi32>, memref<128x4xui8>, memref<4x2xi8>, memref<ui8>, none) -> ()
}

// -----

// A batched right-hand side goes to the same entry point: the runtime pairs
// the batch dimensions itself.
func.func @matmul_integer_batched_b(%a: tensor<2x8x4xui8>, %b: tensor<2x4x2xi8>, %azp: tensor<ui8>, %bzp: tensor<i8>) -> tensor<*xi32> {
  %y = "onnx.MatMulInteger"(%a, %b, %azp, %bzp) : (tensor<2x8x4xui8>, tensor<2x4x2xi8>, tensor<ui8>, tensor<i8>) -> tensor<*xi32>
  return %y : tensor<*xi32>
// CHECK-LABEL:  func.func @matmul_integer_batched_b
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<2x8x2xi32>
// CHECK:        "krnl.call"([[Y]], {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_MatMulInteger", numOfOutput = 1 : si64
// CHECK-SAME:   (memref<2x8x2xi32>, memref<2x8x4xui8>, memref<2x4x2xi8>, memref<ui8>, memref<i8>) -> ()
}

// -----

// narrow_mode = 0: keep the low eight bits, as the CPU lowering does.
func.func @qlinear_matmul(%a: tensor<2x4xui8>, %as: tensor<f32>, %azp: tensor<ui8>, %b: tensor<4x3xui8>, %bs: tensor<f32>, %bzp: tensor<ui8>, %ys: tensor<f32>, %yzp: tensor<ui8>) -> tensor<*xui8> {
  %y = "onnx.QLinearMatMul"(%a, %as, %azp, %b, %bs, %bzp, %ys, %yzp) : (tensor<2x4xui8>, tensor<f32>, tensor<ui8>, tensor<4x3xui8>, tensor<f32>, tensor<ui8>, tensor<f32>, tensor<ui8>) -> tensor<*xui8>
  return %y : tensor<*xui8>
// CHECK-LABEL:  func.func @qlinear_matmul
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<2x3xui8>
// CHECK:        "krnl.call"([[Y]], {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_QLinearMatMul", numOfOutput = 1 : si64
// CHECK-SAME:   narrow_mode = 0 : i64
}
