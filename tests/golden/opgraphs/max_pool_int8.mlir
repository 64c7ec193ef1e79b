module {
  func @tpu_func(%arg0: tensor<4x128x112x112xf32>) -> tensor<4x128x56x56xf32> {
    %0 = "tpu.weight_file"() {filename = "max_pool_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.086520e+00 : f32}} : (tensor<4x128x112x112xf32>) -> tensor<4x128x112x112xf32>
    %q0 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x42756279 : f32, name = "data_quant_i8"} : (tensor<4x128x112x112xf32>) -> tensor<4x128x112x112xsi8>
    %2 = "tpu.pool_max_2d"(%q0) {name = "max_pool", param = {count_include_pad = false, do_relu = false, kernel_h = 2 : i32, kernel_w = 2 : i32, pad_value = 0 : i32, padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 2 : i32, stride_w = 2 : i32}, quant = {mode = "INT8", param_type = "NONE", threshold = 2.086520e+00 : f32}} : (tensor<4x128x112x112xsi8>) -> tensor<4x128x56x56xsi8>
    %q1 = "tpu.quant"(%2) {from = "INT8", to = "NONE", scale = 0x3C85898B : f32, name = "max_pool_dequant"} : (tensor<4x128x56x56xsi8>) -> tensor<4x128x56x56xf32>
    return %q1 : tensor<4x128x56x56xf32>
  }
}
