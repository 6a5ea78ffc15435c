module {
  func.func @main_graph(%X: tensor<128x768xf32>, %B: tensor<768x768xi8>) -> tensor<128x768xf32> {
    %bzp = onnx.Constant dense<0> : tensor<i8>
    %bs = onnx.Constant dense<2.000000e-02> : tensor<f32>
    %xq, %xs, %xzp = "onnx.DynamicQuantizeLinear"(%X) : (tensor<128x768xf32>) -> (tensor<128x768xui8>, tensor<f32>, tensor<ui8>)
    %acc = "onnx.MatMulInteger"(%xq, %B, %xzp, %bzp) : (tensor<128x768xui8>, tensor<768x768xi8>, tensor<ui8>, tensor<i8>) -> tensor<128x768xi32>
    %c = "onnx.Cast"(%acc) {to = f32} : (tensor<128x768xi32>) -> tensor<128x768xf32>
    %s = "onnx.Mul"(%xs, %bs) : (tensor<f32>, tensor<f32>) -> tensor<f32>
    %y = "onnx.Mul"(%c, %s) : (tensor<128x768xf32>, tensor<f32>) -> tensor<128x768xf32>
    return %y : tensor<128x768xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
