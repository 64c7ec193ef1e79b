module {
  func @tpu_func(%arg0: tensor<4x64x227x227xf32>) -> tensor<4x64x227x227xf32> {
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 1.911430e+00 : f32}} : (tensor<4x64x227x227xf32>) -> tensor<4x64x227x227xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 6.696557e+01 : f32, name = "data_quant_i8"} : (tensor<4x64x227x227xf32>) -> tensor<4x64x227x227xsi8>
    %2 = "tpu.reverse"(%q0) {axis = 0 : i32, name = "reverse", quant = {mode = "INT8", param_type = "NONE", threshold = 1.911430e+00 : f32}} : (tensor<4x64x227x227xsi8>) -> tensor<4x64x227x227xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 0x3C74A9BD : f32, name = "reverse_dequant"} : (tensor<4x64x227x227xsi8>) -> tensor<4x64x227x227xf32>
    return %q1 : tensor<4x64x227x227xf32>
  }
}
