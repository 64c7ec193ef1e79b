module {
  func @tpu_func(%arg0: tensor<16x32x64x128xf32>) -> (tensor<32x16x64x128xf32>, tensor<32x16x64x128xf32>, tensor<16x64x32x128xf32>, tensor<16x128x32x64xf32>, tensor<16x64x128x32xf32>, tensor<16x128x64x32xf32>) {
    %1 = "tpu.input"(%arg0) {layer_id = 0 : i32, name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xf32>) -> tensor<16x32x64x128xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 4.313337e+01 : f32, name = "data_quant_i8"} : (tensor<16x32x64x128xf32>) -> tensor<16x32x64x128xsi8>
    %2 = "tpu.permute"(%q0) {name = "permute_1023", order = [1 : i32, 0 : i32, 2 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xsi8>) -> tensor<32x16x64x128xsi8>
    %3 = "tpu.permute"(%2) {name = "permute_0123", order = [0 : i32, 1 : i32, 2 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<32x16x64x128xsi8>) -> tensor<32x16x64x128xsi8>
    %4 = "tpu.permute"(%q0) {name = "permute_0213", order = [0 : i32, 2 : i32, 1 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xsi8>) -> tensor<16x64x32x128xsi8>
    %5 = "tpu.permute"(%q0) {name = "permute_0312", order = [0 : i32, 3 : i32, 1 : i32, 2 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xsi8>) -> tensor<16x128x32x64xsi8>
    %6 = "tpu.permute"(%q0) {name = "permute_0231", order = [0 : i32, 2 : i32, 3 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xsi8>) -> tensor<16x64x128x32xsi8>
    %7 = "tpu.permute"(%q0) {name = "permute_0321", order = [0 : i32, 3 : i32, 2 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.967540e+00 : f32}} : (tensor<16x32x64x128xsi8>) -> tensor<16x128x64x32xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_1023_dequant"} : (tensor<32x16x64x128xsi8>) -> tensor<32x16x64x128xf32>
    %q2 = "tpu.quant"(%3) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_0123_dequant"} : (tensor<32x16x64x128xsi8>) -> tensor<32x16x64x128xf32>
    %q3 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_0213_dequant"} : (tensor<16x64x32x128xsi8>) -> tensor<16x64x32x128xf32>
    %q4 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_0312_dequant"} : (tensor<16x128x32x64xsi8>) -> tensor<16x128x32x64xf32>
    %q5 = "tpu.quant"(%6) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_0231_dequant"} : (tensor<16x64x128x32xsi8>) -> tensor<16x64x128x32xf32>
    %q6 = "tpu.quant"(%7) {from = "INT8", to = "NONE", scale = 0x3CBDEC2D : f32, name = "permute_0321_dequant"} : (tensor<16x128x64x32xsi8>) -> tensor<16x128x64x32xf32>
    return %q1, %q2, %q3, %q4, %q5, %q6 : tensor<32x16x64x128xf32>, tensor<32x16x64x128xf32>, tensor<16x64x32x128xf32>, tensor<16x128x32x64xf32>, tensor<16x64x128x32xf32>, tensor<16x128x64x32xf32>
  }
}
