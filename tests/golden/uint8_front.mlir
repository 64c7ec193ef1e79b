module {
  func @tpu_func(%arg0: tensor<2x3x12x10xui8>) -> tensor<2x24x12x10xsi8> {
    %0 = "tpu.weight_file"() {filename = "uint8_front_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.none"() : () -> none
    %2 = "tpu.input"(%arg0) {name = "input", quant = {mode = "UINT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x3x12x10xui8>) -> tensor<2x3x12x10xui8>
    %3 = "tpu.load_weight"(%0) {name = "x8_table", storage = "INT8"} : (memref<10xf32>) -> tensor<768xf32>
    %4 = "tpu.scale_lut"(%2, %3) {name = "x8", quant = {mode = "INT8", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x3x12x10xui8>, tensor<768xf32>) -> tensor<2x3x12x10xsi8>
    %5 = "tpu.load_weight"(%0) {name = "c1_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<24x3x3x3xf32>
    %6 = "tpu.load_weight"(%0) {name = "c1_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<24xf32>
    %7 = "tpu.load_weight"(%0) {name = "c1_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %8 = "tpu.load_weight"(%0) {name = "c1_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<24xf32>
    %9 = "tpu.conv_2d"(%4, %5, %6, %1, %1, %7, %8) {name = "c1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x3x12x10xsi8>, tensor<24x3x3x3xf32>, tensor<24xf32>, none, none, tensor<24xf32>, tensor<24xf32>) -> tensor<2x24x12x10xsi8>
    return %9 : tensor<2x24x12x10xsi8>
  }
}
