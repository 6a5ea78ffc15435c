module {
  func.func @main_graph(%X: tensor<4x4096xf32>, %B: tensor<4096x11008xi8>, %bs: tensor<11008xf32>) -> tensor<4x11008xf32> {
    %bzp = onnx.Constant dense<0> : tensor<i8>
    %xq, %xs, %xzp = "onnx.DynamicQuantizeLinear"(%X) : (tensor<4x4096xf32>) -> (tensor<4x4096xui8>, tensor<f32>, tensor<ui8>)
    %acc = "onnx.MatMulInteger"(%xq, %B, %xzp, %bzp) : (tensor<4x4096xui8>, tensor<4096x11008xi8>, tensor<ui8>, tensor<i8>) -> tensor<4x11008xi32>
    %c = "onnx.Cast"(%acc) {to = f32} : (tensor<4x11008xi32>) -> tensor<4x11008xf32>
    %s = "onnx.Mul"(%xs, %bs) : (tensor<f32>, tensor<11008xf32>) -> tensor<11008xf32>
    %y = "onnx.Mul"(%c, %s) : (tensor<4x11008xf32>, tensor<11008xf32>) -> tensor<4x11008xf32>
    return %y : tensor<4x11008xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
