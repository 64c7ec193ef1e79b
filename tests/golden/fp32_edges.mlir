module {
  func @tpu_func(%arg0: tensor<2x12x7x6xf32>) -> tensor<2x20x14x12xf32> {
    %0 = "tpu.weight_file"() {filename = "fp32_edges_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.none"() : () -> none
    %2 = "tpu.input"(%arg0) {name = "input", quant = {mode = "NONE", param_type = "NONE", threshold = 0.000000e+00 : f32}} : (tensor<2x12x7x6xf32>) -> tensor<2x12x7x6xf32>
    %3 = "tpu.quant"(%2) {name = "x8", from = "NONE", to = "INT8", scale = 3.175000e+01 : f32} : (tensor<2x12x7x6xf32>) -> tensor<2x12x7x6xsi8>
    %4 = "tpu.load_weight"(%0) {name = "c1_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<16x12x3x3xf32>
    %5 = "tpu.load_weight"(%0) {name = "c1_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<16xf32>
    %6 = "tpu.load_weight"(%0) {name = "c1_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %7 = "tpu.load_weight"(%0) {name = "c1_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<16xf32>
    %8 = "tpu.conv_2d"(%3, %4, %5, %1, %1, %6, %7) {name = "c1", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, do_relu = true} : (tensor<2x12x7x6xsi8>, tensor<16x12x3x3xf32>, tensor<16xf32>, none, none, tensor<16xf32>, tensor<16xf32>) -> tensor<2x16x7x6xsi8>
    %9 = "tpu.load_weight"(%0) {name = "up_filter", storage = "INT8"} : (memref<10xf32>) -> tensor<2880xf32>
    %10 = "tpu.load_weight"(%0) {name = "up_bias", storage = "INT32"} : (memref<10xf32>) -> tensor<20xf32>
    %11 = "tpu.load_weight"(%0) {name = "up_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<20xf32>
    %12 = "tpu.load_weight"(%0) {name = "up_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<20xf32>
    %13 = "tpu.deconv_2d"(%8, %9, %10, %1, %1, %11, %12) {name = "up", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 0.000000e+00 : f32}, param = {dilation_h = 1 : i32, dilation_w = 1 : i32, group = 1 : i32, ins = [], is_dw = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, do_relu = false} : (tensor<2x16x7x6xsi8>, tensor<2880xf32>, tensor<20xf32>, none, none, tensor<20xf32>, tensor<20xf32>) -> tensor<2x20x14x12xsi8>
    %14 = "tpu.quant"(%13) {name = "out", from = "INT8", to = "NONE", scale = 2.070000e-02 : f32} : (tensor<2x20x14x12xsi8>) -> tensor<2x20x14x12xf32>
    return %14 : tensor<2x20x14x12xf32>
  }
}
