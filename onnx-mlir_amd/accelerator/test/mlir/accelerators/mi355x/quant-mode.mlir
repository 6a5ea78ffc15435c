// RUN: onnx-mlir-opt --maccel=MI355X -O3 --enable-fast-math --disable-quantization-zero-point --shape-inference --convert-onnx-to-krnl --canonicalize %s -split-input-file | FileCheck %s
// RUN: onnx-mlir-opt --maccel=MI355X -O3 --shape-inference --convert-onnx-to-krnl --canonicalize %s -split-input-file | FileCheck --check-prefix=DEFAULT %s

// The reference's CPU code for these ops changes with --enable-fast-math (at
// -O3) and --disable-quantization-zero-point; the offloaded ops are told which
// form to compute by a call directly in front of each of them.  The runtime
// applies that call to the very next such op of the thread and to no other, so
// code compiled with default options (DEFAULT) needs no call: an op that none
// precedes computes the default form whatever ran on the thread before.
func.func @quantize_then_dequantize(%x: tensor<64x768xf32>, %s: tensor<f32>, %z: tensor<ui8>) -> tensor<64x768xf32> {
  %q = "onnx.QuantizeLinear"(%x, %s, %z) {axis = 1 : si64, saturate = 1 : si64} : (tensor<64x768xf32>, tensor<f32>, tensor<ui8>) -> tensor<64x768xui8>
  %y = "onnx.DequantizeLinear"(%q, %s, %z) {axis = 1 : si64} : (tensor<64x768xui8>, tensor<f32>, tensor<ui8>) -> tensor<64x768xf32>
  return %y : tensor<64x768xf32>
// CHECK-LABEL:  func.func @quantize_then_dequantize
// CHECK:        [[Q:%.+]] = memref.alloc() {{.*}}: memref<64x768xui8>
// CHECK:        "krnl.call"([[Q]]) {funcName = "om_mi355x_SetQuantMode", mode = 3 : i64, numOfOutput = 1 : si64}
// CHECK:        "krnl.call"([[Q]], {{.*}}) {axis = 1 : i64, funcName = "om_mi355x_QuantizeLinear", numOfOutput = 1 : si64, saturate = 1 : i64}
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<64x768xf32>
// CHECK:        "krnl.call"([[Y]]) {funcName = "om_mi355x_SetQuantMode", mode = 3 : i64, numOfOutput = 1 : si64}
// CHECK:        "krnl.call"([[Y]], [[Q]], {{.*}}) {axis = 1 : i64, funcName = "om_mi355x_DequantizeLinear", numOfOutput = 1 : si64}
// DEFAULT-LABEL: func.func @quantize_then_dequantize
// DEFAULT-NOT:   om_mi355x_SetQuantMode
// DEFAULT:       funcName = "om_mi355x_QuantizeLinear"
// DEFAULT-NOT:   om_mi355x_SetQuantMode
// DEFAULT:       funcName = "om_mi355x_DequantizeLinear"
}

// -----

func.func @dynamic_quantize(%x: tensor<128x768xf32>) -> (tensor<128x768xui8>, tensor<f32>, tensor<ui8>) {
  %q, %s, %z = "onnx.DynamicQuantizeLinear"(%x) : (tensor<128x768xf32>) -> (tensor<128x768xui8>, tensor<f32>, tensor<ui8>)
  return %q, %s, %z : tensor<128x768xui8>, tensor<f32>, tensor<ui8>
// CHECK-LABEL:  func.func @dynamic_quantize
// CHECK:        [[Q:%.+]] = memref.alloc() {{.*}}: memref<128x768xui8>
// CHECK:        "krnl.call"([[Q]]) {funcName = "om_mi355x_SetQuantMode", mode = 3 : i64, numOfOutput = 1 : si64}
// CHECK:        "krnl.call"([[Q]], {{.*}}) {funcName = "om_mi355x_DynamicQuantizeLinear", numOfOutput = 3 : si64}
// DEFAULT-LABEL: func.func @dynamic_quantize
// DEFAULT-NOT:   om_mi355x_SetQuantMode
}
