module {
  func @tpu_func(%arg0: tensor<1x3x1x22400xf32>) -> tensor<1x1x1x5600xf32> {
    %0 = "tpu.weight_file"() {filename = "conv_large_w_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.546720e+00 : f32}} : (tensor<1x3x1x22400xf32>) -> tensor<1x3x1x22400xf32>
    %2 = "tpu.load_weight"(%0) {name = "filter_0.866710_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<32x3x3x3xf32>
    %3 = "tpu.load_weight"(%0) {name = "bias_0.866710_quant", storage = "INT32"} : (memref<10xf32>) -> tensor<32xf32>
    %4 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "conv_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<32xf32>
    %q1 = "tpu.load_weight"(%0) {name = "conv_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<32xf32>
    %q4 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x42490AFC : f32, name = "data_quant_i8"} : (tensor<1x3x1x22400xf32>) -> tensor<1x3x1x22400xsi8>
    %5 = "tpu.conv_2d"(%q4, %2, %3, %4, %4, %q0, %q1) {name = "conv", param = {dilation_h = 1 : i32, dilation_w = 1 : i32, do_relu = false, group = 1 : i32, ins = [], is_dw = false, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 8.667100e-01 : f32}} : (tensor<1x3x1x22400xsi8>, tensor<32x3x3x3xf32>, tensor<32xf32>, none, none, tensor<32xf32>, tensor<32xf32>) -> tensor<1x32x1x11200xsi8>
    %6 = "tpu.load_weight"(%0) {name = "filter_1_1.310690_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<1x32x3x3xf32>
    %7 = "tpu.load_weight"(%0) {name = "bias_1_1.310690_quant", storage = "INT32"} : (memref<10xf32>) -> tensor<1xf32>
    %8 = "tpu.none"() : () -> none
    %q2 = "tpu.load_weight"(%0) {name = "conv_1_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %q3 = "tpu.load_weight"(%0) {name = "conv_1_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %9 = "tpu.conv_2d"(%5, %6, %7, %8, %8, %q2, %q3) {name = "conv_1", param = {dilation_h = 1 : i32, dilation_w = 1 : i32, do_relu = false, group = 1 : i32, ins = [], is_dw = false, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 1.310690e+00 : f32}} : (tensor<1x32x1x11200xsi8>, tensor<1x32x3x3xf32>, tensor<1xf32>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<1x1x1x5600xsi8>
    %q5 = "tpu.quant"(%9) {from = "INT8", to = "NONE", scale = 0x3C27C4B1 : f32, name = "conv_1_dequant"} : (tensor<1x1x1x5600xsi8>) -> tensor<1x1x1x5600xf32>
    return %q5 : tensor<1x1x1x5600xf32>
  }
}
