module {
  func.func @main_graph(%X: tensor<8192x32768xf32>, %s: tensor<f32>, %zp: tensor<ui8>) -> (tensor<8192x32768xui8>, tensor<8192x32768xf32>, tensor<8192x32768xui8>, tensor<f32>, tensor<ui8>) {
    %q = "onnx.QuantizeLinear"(%X, %s, %zp) {axis = 1 : si64} : (tensor<8192x32768xf32>, tensor<f32>, tensor<ui8>) -> tensor<8192x32768xui8>
    %d = "onnx.DequantizeLinear"(%q, %s, %zp) {axis = 1 : si64} : (tensor<8192x32768xui8>, tensor<f32>, tensor<ui8>) -> tensor<8192x32768xf32>
    %dq, %ds, %dzp = "onnx.DynamicQuantizeLinear"(%X) : (tensor<8192x32768xf32>) -> (tensor<8192x32768xui8>, tensor<f32>, tensor<ui8>)
    return %q, %d, %dq, %ds, %dzp : tensor<8192x32768xui8>, tensor<8192x32768xf32>, tensor<8192x32768xui8>, tensor<f32>, tensor<ui8>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
