module {
  func @tpu_func(%arg0: tensor<1x16x64x128xf32>) -> tensor<1x1x128x256xf32> {
    %0 = "tpu.weight_file"() {filename = "deconv_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data0", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 1.312970e+00 : f32}} : (tensor<1x16x64x128xf32>) -> tensor<1x16x64x128xf32>
    %2 = "tpu.load_weight"(%0) {name = "deconv_0_3.985000_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<1x16x2x2xf32>
    %3 = "tpu.load_weight"(%0) {name = "deconv_1_3.985000_quant", storage = "INT32"} : (memref<10xf32>) -> tensor<1xf32>
    %4 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "deconv_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "deconv_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 9.748890e+01 : f32, name = "data0_quant_i8"} : (tensor<1x16x64x128xf32>) -> tensor<1x16x64x128xsi8>
    %5 = "tpu.deconv_2d"(%q2, %2, %3, %4, %4, %q0, %q1) {name = "deconv", param = {dilation_h = 1 : i32, dilation_w = 1 : i32, do_relu = false, group = 1 : i32, ins = [], is_dw = false, pad_value = 0 : i32, padding = "VALID", padding_b = 0 : i32, padding_l = 0 : i32, padding_r = 0 : i32, padding_t = 0 : i32, stride_h = 2 : i32, stride_w = 2 : i32, with_bias = true}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 3.985000e+00 : f32}} : (tensor<1x16x64x128xsi8>, tensor<1x16x2x2xf32>, tensor<1xf32>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<1x1x128x256xsi8>
    %q3 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3CFF0A3D : f32, name = "deconv_dequant"} : (tensor<1x1x128x256xsi8>) -> tensor<1x1x128x256xf32>
    return %q3 : tensor<1x1x128x256xf32>
  }
}
