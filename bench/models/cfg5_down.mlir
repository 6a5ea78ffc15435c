module {
  func.func @main_graph(%X: tensor<2048x11008xf32>, %B: tensor<11008x4096xi8>, %bs: tensor<4096xf32>) -> tensor<2048x4096xf32> {
    %bzp = onnx.Constant dense<0> : tensor<i8>
    %xq, %xs, %xzp = "onnx.DynamicQuantizeLinear"(%X) : (tensor<2048x11008xf32>) -> (tensor<2048x11008xui8>, tensor<f32>, tensor<ui8>)
    %acc = "onnx.MatMulInteger"(%xq, %B, %xzp, %bzp) : (tensor<2048x11008xui8>, tensor<11008x4096xi8>, tensor<ui8>, tensor<i8>) -> tensor<2048x4096xi32>
    %c = "onnx.Cast"(%acc) {to = f32} : (tensor<2048x4096xi32>) -> tensor<2048x4096xf32>
    %s = "onnx.Mul"(%xs, %bs) : (tensor<f32>, tensor<4096xf32>) -> tensor<4096xf32>
    %y = "onnx.Mul"(%c, %s) : (tensor<2048x4096xf32>, tensor<4096xf32>) -> tensor<2048x4096xf32>
    return %y : tensor<2048x4096xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
