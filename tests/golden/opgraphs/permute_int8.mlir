module {
  func @tpu_func(%arg0: tensor<16x16x16x16xf32>) -> (tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>) {
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xf32>) -> tensor<16x16x16x16xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 5.221506e+01 : f32, name = "data_quant_i8"} : (tensor<16x16x16x16xf32>) -> tensor<16x16x16x16xsi8>
    %2 = "tpu.permute"(%q0) {name = "permute_1023", order = [1 : i32, 0 : i32, 2 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %3 = "tpu.permute"(%2) {name = "permute_0123", order = [0 : i32, 1 : i32, 2 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %4 = "tpu.permute"(%q0) {name = "permute_0213", order = [0 : i32, 2 : i32, 1 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %5 = "tpu.permute"(%q0) {name = "permute_2013", order = [2 : i32, 0 : i32, 1 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %6 = "tpu.permute"(%q0) {name = "permute_2103", order = [2 : i32, 1 : i32, 0 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %7 = "tpu.permute"(%q0) {name = "permute_1203", order = [1 : i32, 2 : i32, 0 : i32, 3 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %8 = "tpu.permute"(%q0) {name = "permute_0312", order = [0 : i32, 3 : i32, 1 : i32, 2 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %9 = "tpu.permute"(%q0) {name = "permute_0321", order = [0 : i32, 3 : i32, 2 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %10 = "tpu.permute"(%q0) {name = "permute_0231", order = [0 : i32, 2 : i32, 3 : i32, 1 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %11 = "tpu.permute"(%q0) {name = "permute_0132", order = [0 : i32, 1 : i32, 3 : i32, 2 : i32], quant = {mode = "INT8", param_type = "NONE", threshold = 2.451400e+00 : f32}} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_1023_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q2 = "tpu.quant"(%3) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0123_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q3 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0213_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q4 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_2013_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q5 = "tpu.quant"(%6) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_2103_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q6 = "tpu.quant"(%7) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_1203_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q7 = "tpu.quant"(%8) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0312_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q8 = "tpu.quant"(%9) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0321_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q9 = "tpu.quant"(%10) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0231_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    %q10 = "tpu.quant"(%11) {from = "INT8", to = "NONE", scale = 0x3C9CE3BD : f32, name = "permute_0132_dequant"} : (tensor<16x16x16x16xsi8>) -> tensor<16x16x16x16xf32>
    return %q1, %q2, %q3, %q4, %q5, %q6, %q7, %q8, %q9, %q10 : tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>, tensor<16x16x16x16xf32>
  }
}
