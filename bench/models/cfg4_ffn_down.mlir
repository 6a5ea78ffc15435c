module {
  func.func @main_graph(%X: tensor<4096x3072xf32>, %B: tensor<3072x768xi8>, %bs: tensor<768xf32>) -> tensor<4096x768xf32> {
    %bzp = onnx.Constant dense<0> : tensor<i8>
    %xq, %xs, %xzp = "onnx.DynamicQuantizeLinear"(%X) : (tensor<4096x3072xf32>) -> (tensor<4096x3072xui8>, tensor<f32>, tensor<ui8>)
    %acc = "onnx.MatMulInteger"(%xq, %B, %xzp, %bzp) : (tensor<4096x3072xui8>, tensor<3072x768xi8>, tensor<ui8>, tensor<i8>) -> tensor<4096x768xi32>
    %c = "onnx.Cast"(%acc) {to = f32} : (tensor<4096x768xi32>) -> tensor<4096x768xf32>
    %s = "onnx.Mul"(%xs, %bs) : (tensor<f32>, tensor<768xf32>) -> tensor<768xf32>
    %y = "onnx.Mul"(%c, %s) : (tensor<4096x768xf32>, tensor<768xf32>) -> tensor<4096x768xf32>
    return %y : tensor<4096x768xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
