module {
  func @tpu_func(%arg0: tensor<64x3x256x256xf32>) -> (tensor<64x3x256x256xf32>, tensor<64x3x256x256xf32>) {
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.825330e+00 : f32}} : (tensor<64x3x256x256xf32>) -> tensor<64x3x256x256xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x423537C0 : f32, name = "data_quant_i8"} : (tensor<64x3x256x256xf32>) -> tensor<64x3x256x256xsi8>
    %2 = "tpu.swap_channel"(%q0) {name = "older201", channel_order = [2 : i32, 0 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.825330e+00 : f32}} : (tensor<64x3x256x256xsi8>) -> tensor<64x3x256x256xsi8>
    %3 = "tpu.swap_channel"(%q0) {name = "older120", channel_order = [1 : i32, 2 : i32, 0 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.825330e+00 : f32}} : (tensor<64x3x256x256xsi8>) -> tensor<64x3x256x256xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 2.207289e-02 : f32, name = "older201_dequant"} : (tensor<64x3x256x256xsi8>) -> tensor<64x3x256x256xf32>
    %q2 = "tpu.quant"(%3) {from = "INT8", to = "NONE", scale = 2.207289e-02 : f32, name = "older120_dequant"} : (tensor<64x3x256x256xsi8>) -> tensor<64x3x256x256xf32>
    return %q1, %q2 : tensor<64x3x256x256xf32>, tensor<64x3x256x256xf32>
  }
}
