// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --recompose-qdq-matmul-for-mi355x --canonicalize %s -split-input-file | FileCheck %s
// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --recompose-qdq-matmul-for-mi355x="per-column-only=true" --canonicalize %s -split-input-file | FileCheck --check-prefix=COLUMN %s
// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --recompose-qdq-matmul-for-mi355x --convert-onnx-to-krnl --canonicalize %s -split-input-file | FileCheck --check-prefix=KRNL %s

// A linear layer of a statically quantized (QDQ) model whose weights have one
// scale per output channel: DequantizeLinear {axis = 1} on the weights, a
// float MatMul, QuantizeLinear.  The chain becomes onnx.QLinearMatMul with the
// 1-D scale and zero point as b_scale / b_zero_point, which the accelerator
// lowers to one call; the int8 weights are what the kernel reads.
func.func @per_column_weights(%a: tensor<512x1024xui8>, %as: tensor<f32>, %az: tensor<ui8>, %w: tensor<1024x4096xi8>, %ws: tensor<4096xf32>, %wz: tensor<4096xi8>, %ys: tensor<f32>, %yz: tensor<ui8>) -> tensor<512x4096xui8> {
  %af = "onnx.DequantizeLinear"(%a, %as, %az) {axis = 1 : si64} : (tensor<512x1024xui8>, tensor<f32>, tensor<ui8>) -> tensor<512x1024xf32>
  %wf = "onnx.DequantizeLinear"(%w, %ws, %wz) {axis = 1 : si64} : (tensor<1024x4096xi8>, tensor<4096xf32>, tensor<4096xi8>) -> tensor<1024x4096xf32>
  %yf = "onnx.MatMul"(%af, %wf) : (tensor<512x1024xf32>, tensor<1024x4096xf32>) -> tensor<512x4096xf32>
  %y = "onnx.QuantizeLinear"(%yf, %ys, %yz) {axis = 1 : si64, saturate = 1 : si64} : (tensor<512x4096xf32>, tensor<f32>, tensor<ui8>) -> tensor<512x4096xui8>
  return %y : tensor<512x4096xui8>
// CHECK-LABEL:  func.func @per_column_weights
// CHECK-SAME:   ([[A:%.+]]: tensor<512x1024xui8>, [[AS:%.+]]: tensor<f32>, [[AZ:%.+]]: tensor<ui8>, [[W:%.+]]: tensor<1024x4096xi8>, [[WS:%.+]]: tensor<4096xf32>, [[WZ:%.+]]: tensor<4096xi8>, [[YS:%.+]]: tensor<f32>, [[YZ:%.+]]: tensor<ui8>)
// CHECK-NOT:    onnx.DequantizeLinear
// CHECK-NOT:    onnx.MatMul
// CHECK:        [[Y:%.+]] = "onnx.QLinearMatMul"([[A]], [[AS]], [[AZ]], [[W]], [[WS]], [[WZ]], [[YS]], [[YZ]])
// CHECK-NOT:    onnx.QuantizeLinear
// CHECK:        return [[Y]]
// COLUMN-LABEL: func.func @per_column_weights
// COLUMN:       "onnx.QLinearMatMul"
// KRNL-LABEL:   func.func @per_column_weights
// KRNL:         [[Y:%.+]] = memref.alloc() {{.*}}: memref<512x4096xui8>
// KRNL:         "krnl.call"([[Y]], {{.*}}) {funcName = "om_mi355x_QLinearMatMul", narrow_mode = 0 : i64, numOfOutput = 1 : si64}
}

// -----

// Weights without a zero point (symmetric): QLinearMatMul's zero points are
// required, so zeros of the weights' type and the scale's shape are made.
func.func @symmetric_weights(%a: tensor<64x768xi8>, %as: tensor<f32>, %az: tensor<i8>, %w: tensor<768x3072xi8>, %ws: tensor<3072xf32>, %ys: tensor<f32>, %yz: tensor<i8>) -> tensor<64x3072xi8> {
  %none = "onnx.NoValue"() {value} : () -> none
  %af = "onnx.DequantizeLinear"(%a, %as, %az) {axis = 1 : si64} : (tensor<64x768xi8>, tensor<f32>, tensor<i8>) -> tensor<64x768xf32>
  %wf = "onnx.DequantizeLinear"(%w, %ws, %none) {axis = -1 : si64} : (tensor<768x3072xi8>, tensor<3072xf32>, none) -> tensor<768x3072xf32>
  %yf = "onnx.MatMul"(%af, %wf) : (tensor<64x768xf32>, tensor<768x3072xf32>) -> tensor<64x3072xf32>
  %y = "onnx.QuantizeLinear"(%yf, %ys, %yz) {axis = 1 : si64, saturate = 1 : si64} : (tensor<64x3072xf32>, tensor<f32>, tensor<i8>) -> tensor<64x3072xi8>
  return %y : tensor<64x3072xi8>
// CHECK-LABEL:  func.func @symmetric_weights
// CHECK:        [[ZERO:%.+]] = onnx.Constant dense<0> : tensor<3072xi8>
// CHECK:        [[Y:%.+]] = "onnx.QLinearMatMul"(%arg0, %arg1, %arg2, %arg3, %arg4, [[ZERO]], %arg5, %arg6)
// CHECK:        return [[Y]]
}

// -----

// One scale for all of W: recomposed as well (as the ONNX dialect's own
// recomposition would), unless the pass is told to add only what that one
// does not do.
func.func @per_tensor_weights(%a: tensor<64x768xui8>, %as: tensor<f32>, %az: tensor<ui8>, %w: tensor<768x768xi8>, %ws: tensor<f32>, %wz: tensor<i8>, %ys: tensor<f32>, %yz: tensor<ui8>) -> tensor<64x768xui8> {
  %af = "onnx.DequantizeLinear"(%a, %as, %az) {axis = 1 : si64} : (tensor<64x768xui8>, tensor<f32>, tensor<ui8>) -> tensor<64x768xf32>
  %wf = "onnx.DequantizeLinear"(%w, %ws, %wz) {axis = 1 : si64} : (tensor<768x768xi8>, tensor<f32>, tensor<i8>) -> tensor<768x768xf32>
  %yf = "onnx.MatMul"(%af, %wf) : (tensor<64x768xf32>, tensor<768x768xf32>) -> tensor<64x768xf32>
  %y = "onnx.QuantizeLinear"(%yf, %ys, %yz) {axis = 1 : si64, saturate = 1 : si64} : (tensor<64x768xf32>, tensor<f32>, tensor<ui8>) -> tensor<64x768xui8>
  return %y : tensor<64x768xui8>
// CHECK-LABEL:  func.func @per_tensor_weights
// CHECK:        "onnx.QLinearMatMul"
// CHECK-NOT:    onnx.MatMul
// COLUMN-LABEL: func.func @per_tensor_weights
// COLUMN-NOT:   onnx.QLinearMatMul
// COLUMN:       "onnx.MatMul"
}

// -----

// Not a scale per output column: weights quantized per row (axis = 0), and a
// float product that something else reads too.  Both stay as they are.
func.func @left_alone(%a: tensor<64x768xui8>, %as: tensor<f32>, %az: tensor<ui8>, %w: tensor<768x768xi8>, %wsr: tensor<768xf32>, %wzr: tensor<768xi8>, %ys: tensor<f32>, %yz: tensor<ui8>) -> (tensor<64x768xui8>, tensor<64x768xui8>, tensor<64x768xf32>) {
  %af = "onnx.DequantizeLinear"(%a, %as, %az) {axis = 1 : si64} : (tensor<64x768xui8>, tensor<f32>, tensor<ui8>) -> tensor<64x768xf32>
  %wf = "onnx.DequantizeLinear"(%w, %wsr, %wzr) {axis = 0 : si64} : (tensor<768x768xi8>, tensor<768xf32>, tensor<768xi8>) -> tensor<768x768xf32>
  %yf = "onnx.MatMul"(%af, %wf) : (tensor<64x768xf32>, tensor<768x768xf32>) -> tensor<64x768xf32>
  %y = "onnx.QuantizeLinear"(%yf, %ys, %yz) {axis = 1 : si64, saturate = 1 : si64} : (tensor<64x768xf32>, tensor<f32>, tensor<ui8>) -> tensor<64x768xui8>
  %af2 = "onnx.DequantizeLinear"(%a, %as, %az) {axis = 1 : si64} : (tensor<64x768xui8>, tensor<f32>, tensor<ui8>) -> tensor<64x768xf32>
  %wf2 = "onnx.DequantizeLinear"(%w, %wsr, %wzr) {axis = 1 : si64} : (tensor<768x768xi8>, tensor<768xf32>, tensor<768xi8>) -> tensor<768x768xf32>
  %yf2 = "onnx.MatMul"(%af2, %wf2) : (tensor<64x768xf32>, tensor<768x768xf32>) -> tensor<64x768xf32>
  %y2 = "onnx.QuantizeLinear"(%yf2, %ys, %yz) {axis = 1 : si64, saturate = 1 : si64} : (tensor<64x768xf32>, tensor<f32>, tensor<ui8>) -> tensor<64x768xui8>
  return %y, %y2, %yf2 : tensor<64x768xui8>, tensor<64x768xui8>, tensor<64x768xf32>
// CHECK-LABEL:  func.func @left_alone
// CHECK-NOT:    onnx.QLinearMatMul
// CHECK-COUNT-2: "onnx.MatMul"
}
