module {
  func.func @main_graph(%X: tensor<8192x32768xf32>, %s: tensor<32768xf32>, %zp: tensor<32768xui8>) -> (tensor<8192x32768xui8>, tensor<8192x32768xf32>) {
    %lo = onnx.Constant dense<0.000000e+00> : tensor<f32>
    %hi = onnx.Constant dense<2.550000e+02> : tensor<f32>
    %zf = "onnx.Cast"(%zp) {to = f32} : (tensor<32768xui8>) -> tensor<32768xf32>
    %v = "onnx.Div"(%X, %s) : (tensor<8192x32768xf32>, tensor<32768xf32>) -> tensor<8192x32768xf32>
    %r = "onnx.Round"(%v) : (tensor<8192x32768xf32>) -> tensor<8192x32768xf32>
    %a = "onnx.Add"(%r, %zf) : (tensor<8192x32768xf32>, tensor<32768xf32>) -> tensor<8192x32768xf32>
    %c = "onnx.Clip"(%a, %lo, %hi) : (tensor<8192x32768xf32>, tensor<f32>, tensor<f32>) -> tensor<8192x32768xf32>
    %q = "onnx.Cast"(%c) {to = ui8} : (tensor<8192x32768xf32>) -> tensor<8192x32768xui8>
    %qf = "onnx.Cast"(%q) {to = f32} : (tensor<8192x32768xui8>) -> tensor<8192x32768xf32>
    %m = "onnx.Sub"(%qf, %zf) : (tensor<8192x32768xf32>, tensor<32768xf32>) -> tensor<8192x32768xf32>
    %d = "onnx.Mul"(%m, %s) : (tensor<8192x32768xf32>, tensor<32768xf32>) -> tensor<8192x32768xf32>
    return %q, %d : tensor<8192x32768xui8>, tensor<8192x32768xf32>
  }
  "onnx.EntryPoint"() {func = @main_graph} : () -> ()
}
