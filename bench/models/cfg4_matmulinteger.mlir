module {
  func.func @main_graph(%A: tensor<4096x768xui8>, %B: tensor<768x3072xi8>, %azp: tensor<ui8>, %as: tensor<f32>, %bs: tensor<3072xf32>) -> tensor<4096x3072xf32> {
    %none = "onnx.NoValue"() {value} : () -> none
    %acc = "onnx.MatMulInteger"(%A, %B, %azp, %none) : (tensor<4096x768xui8>, tensor<768x3072xi8>, tensor<ui8>, none) -> tensor<4096x3072xi32>
    %c = "onnx.Cast"(%acc) {to = f32} : (tensor<4096x3072xi32>) -> tensor<4096x3072xf32>
    %s = "onnx.Mul"(%as, %bs) : (tensor<f32>, tensor<3072xf32>) -> tensor<3072xf32>
    %y = "onnx.Mul"(%c, %s) : (tensor<4096x3072xf32>, tensor<3072xf32>) -> tensor<4096x3072xf32>
    return %y : tensor<4096x3072xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
