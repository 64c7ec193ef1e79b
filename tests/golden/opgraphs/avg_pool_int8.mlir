module {
  func @tpu_func(%arg0: tensor<1x1024x17x17xf32>) -> tensor<1x1024x17x17xf32> {
    %0 = "tpu.weight_file"() {filename = "avg_pool_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.285030e+00 : f32}} : (tensor<1x1024x17x17xf32>) -> tensor<1x1024x17x17xf32>
    %2 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "inception_b4_pool_ave_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "inception_b4_pool_ave_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x4260112D : f32, name = "data_quant_i8"} : (tensor<1x1024x17x17xf32>) -> tensor<1x1024x17x17xsi8>
    %3 = "tpu.pool_avg_2d"(%q2, %2, %2, %q0, %q1) {name = "inception_b4_pool_ave", param = {count_include_pad = true, do_relu = false, kernel_h = 3 : i32, kernel_w = 3 : i32, pad_value = 0 : i32, padding_b = 1 : i32, padding_l = 1 : i32, padding_r = 1 : i32, padding_t = 1 : i32, stride_h = 1 : i32, stride_w = 1 : i32}, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.161920e+00 : f32}} : (tensor<1x1024x17x17xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<1x1024x17x17xsi8>
    %q3 = "tpu.quant"(%3) {from = "INT8", to = "NONE", scale = 2.470250e-02 : f32, name = "inception_b4_pool_ave_dequant"} : (tensor<1x1024x17x17xsi8>) -> tensor<1x1024x17x17xf32>
    return %q3 : tensor<1x1024x17x17xf32>
  }
}
