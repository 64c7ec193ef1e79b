module {
  func @tpu_func(%arg0: tensor<1x64x288x512xf32>) -> tensor<1x1x288x512xf32> {
    %0 = "tpu.weight_file"() {filename = "conv_1_oc_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 1.733710e+00 : f32}} : (tensor<1x64x288x512xf32>) -> tensor<1x64x288x512xf32>
    %2 = "tpu.load_weight"(%0) {name = "filter_0.807310_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<1x64x3x3xf32>
    %3 = "tpu.load_weight"(%0) {name = "bias_0.807310_quant", storage = "INT32"} : (memref<10xf32>) -> tensor<1xf32>
    %4 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "cls_rshift", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "cls_multiplier", storage = "UINT32"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 7.383011e+01 : f32, name = "data_quant_i8"} : (tensor<1x64x288x512xf32>) -> tensor<1x64x288x512xsi8>
    %5 = "tpu.conv_2d"(%q2, %2, %3, %4, %4, %q0, %q1) {name = "cls", param = {dilation_h = 1 : i32, dilation_w = 1 : i32, do_relu = false, group = 1 : i32, ins = [], is_dw = false, pad_value = 0 : i32, padding = "SAME", padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32, with_bias = true}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 8.073100e-01 : f32}} : (tensor<1x64x288x512xsi8>, tensor<1x64x3x3xf32>, tensor<1xf32>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<1x1x288x512xsi8>
    %q3 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3BCEABDE : f32, name = "cls_dequant"} : (tensor<1x1x288x512xsi8>) -> tensor<1x1x288x512xf32>
    return %q3 : tensor<1x1x288x512xf32>
  }
}
