// RUN: onnx-mlir-opt --maccel=MI355X --shape-inference --fuse-quantized-matmul-for-mi355x --convert-onnx-to-krnl --canonicalize %s | FileCheck %s

// Dynamic batch: the result is allocated from dim 0 of x and dim 1 of w.
func.func @whole_layer_dynamic(%x: tensor<?x768xf32>, %ws: tensor<f32>) -> tensor<*xf32> {
  %w = onnx.Constant dense<1> : tensor<768x64xi8>
  %none = "onnx.NoValue"() {value} : () -> none
  %aq, %as, %azp = "onnx.DynamicQuantizeLinear"(%x) : (tensor<?x768xf32>) -> (tensor<*xui8>, tensor<*xf32>, tensor<*xui8>)
  %acc = "onnx.MatMulInteger"(%aq, %w, %azp, %none) : (tensor<*xui8>, tensor<768x64xi8>, tensor<*xui8>, none) -> tensor<*xi32>
  %f = "onnx.Cast"(%acc) {to = f32} : (tensor<*xi32>) -> tensor<*xf32>
  %s = "onnx.Mul"(%as, %ws) : (tensor<*xf32>, tensor<f32>) -> tensor<*xf32>
  %y = "onnx.Mul"(%f, %s) : (tensor<*xf32>, tensor<*xf32>) -> tensor<*xf32>
  return %y : tensor<*xf32>
// CHECK-LABEL:  func.func @whole_layer_dynamic
// CHECK-SAME:   ([[X:%.+]]: memref<?x768xf32>, [[WS:%.+]]: memref<f32>) -> memref<?x64xf32>
// CHECK-DAG:    [[W:%.+]] = "krnl.global"()
// CHECK-DAG:    [[M:%.+]] = memref.dim [[X]]
// CHECK:        [[Y:%.+]] = memref.alloc([[M]]) {{.*}}: memref<?x64xf32>
// CHECK:        "krnl.call"([[W]])
// CHECK-SAME:   funcName = "om_mi355x_MarkConstant"
// CHECK:        "krnl.call"([[Y]], [[X]], [[W]], {{%.+}}, [[WS]], {{%.+}})
// CHECK-SAME:   activation = 0 : i64
// CHECK-SAME:   funcName = "om_mi355x_DynQuantMatMulDequant", numOfOutput = 1 : si64
// CHECK-SAME:   (memref<?x64xf32>, memref<?x768xf32>, memref<768x64xi8>, none, memref<f32>, none) -> ()
// CHECK-NOT:    krnl.iterate
}
