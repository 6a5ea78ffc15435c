// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --convert-onnx-to-krnl --canonicalize --keep-buffers-on-mi355x %s -split-input-file | FileCheck %s

// The 8-bit activation and its zero point go from one offloaded op to the
// next and nowhere else: both are backed by GPU memory from the allocation to
// just after the matmul.  The scale is also read by the CPU multiplication,
// and the accumulator by the CPU cast, so both stay ordinary host buffers.
func.func @between_two_calls(%x: tensor<256x64xf32>, %ws: tensor<f32>) -> tensor<*xf32> {
  %w = onnx.Constant dense<1> : tensor<64x32xi8>
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<256x64xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<64x32xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<f32>) -> tensor<*xf32>
  %y = "onnx.Add"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @between_two_calls
// CHECK-DAG:    [[AQ:%.+]] = memref.alloc() {{.*}}: memref<256x64xui8>
// CHECK-DAG:    [[AS:%.+]] = memref.alloc() {{.*}}: memref<f32>
// CHECK-DAG:    [[AZP:%.+]] = memref.alloc() {{.*}}: memref<ui8>
// CHECK-DAG:    "krnl.call"([[AQ]]) {funcName = "om_mi355x_KeepOnDevice", numOfOutput = 1 : si64}
// CHECK-DAG:    "krnl.call"([[AZP]]) {funcName = "om_mi355x_KeepOnDevice", numOfOutput = 1 : si64}
// CHECK-NOT:    "krnl.call"([[AS]]) {funcName = "om_mi355x_KeepOnDevice"
// CHECK:        "krnl.call"([[AQ]], [[AS]], [[AZP]], {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_DynamicQuantizeLinear"
// CHECK:        [[ACC:%.+]] = memref.alloc() {{.*}}: memref<256x32xi32>
// CHECK-NOT:    "om_mi355x_KeepOnDevice"
// CHECK:        "krnl.call"([[ACC]], [[AQ]], {{%.+}}, [[AZP]], {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_MatMulInteger"
// CHECK-DAG:    "krnl.call"([[AQ]]) {funcName = "om_mi355x_Release", numOfOutput = 1 : si64}
// CHECK-DAG:    "krnl.call"([[AZP]]) {funcName = "om_mi355x_Release", numOfOutput = 1 : si64}
// CHECK-NOT:    "krnl.call"([[ACC]]) {funcName = "om_mi355x_Release"
}

// -----

// A result that is returned to the caller is never backed.
func.func @returned_result(%x: tensor<256x64xf32>, %s: tensor<f32>, %z: tensor<ui8>) -> tensor<*xf32> {
  %q = "onnx.QuantizeLinear"(%x, %s, %z) {axis = 1 : si64} : (tensor<256x64xf32>, tensor<f32>, tensor<ui8>) -> tensor<*xui8>
  %y = "onnx.DequantizeLinear"(%q, %s, %z) {axis = 1 : si64} : (tensor<*xui8>, tensor<f32>, tensor<ui8>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @returned_result
// CHECK:        [[Q:%.+]] = memref.alloc() {{.*}}: memref<256x64xui8>
// CHECK-NEXT:   "krnl.call"([[Q]]) {funcName = "om_mi355x_KeepOnDevice", numOfOutput = 1 : si64}
// CHECK:        "krnl.call"([[Q]], {{%.+}}, {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_QuantizeLinear"
// CHECK:        [[Y:%.+]] = memref.alloc() {{.*}}: memref<256x64xf32>
// CHECK-NOT:    "krnl.call"([[Y]]) {funcName = "om_mi355x_KeepOnDevice"
// CHECK:        "krnl.call"([[Y]], [[Q]], {{%.+}}, {{%.+}})
// CHECK-SAME:   funcName = "om_mi355x_DequantizeLinear"
// CHECK-NEXT:   "krnl.call"([[Q]]) {funcName = "om_mi355x_Release", numOfOutput = 1 : si64}
// CHECK:        return [[Y]]
}
