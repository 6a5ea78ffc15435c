module {
  func.func @main_graph(%A: tensor<512x1024xui8>, %B: tensor<1024x4096xui8>) -> tensor<512x4096xui8> {
    %as = onnx.Constant dense<1.000000e-02> : tensor<f32>
    %azp = onnx.Constant dense<128> : tensor<ui8>
    %bs = onnx.Constant dense<5.000000e-03> : tensor<f32>
    %bzp = onnx.Constant dense<120> : tensor<ui8>
    %ys = onnx.Constant dense<5.000000e-01> : tensor<f32>
    %yzp = onnx.Constant dense<0> : tensor<ui8>
    %y = "onnx.QLinearMatMul"(%A, %as, %azp, %B, %bs, %bzp, %ys, %yzp) : (tensor<512x1024xui8>, tensor<f32>, tensor<ui8>, tensor<1024x4096xui8>, tensor<f32>, tensor<ui8>, tensor<f32>, tensor<ui8>) -> tensor<512x4096xui8>
    return %y : tensor<512x4096xui8>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
