module {
  func @tpu_func(%arg0: tensor<16x256x32x32xf32>, %arg1: tensor<16x1x32x32xf32>) -> (tensor<16x256x32x32xf32>, tensor<16x256x32x32xf32>, tensor<16x256x32x32xf32>) {
    %0 = "tpu.weight_file"() {filename = "broadcast_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data0", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.374550e+00 : f32}} : (tensor<16x256x32x32xf32>) -> tensor<16x256x32x32xf32>
    %2 = "tpu.input"(%arg1) {name = "data1", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.927510e+00 : f32}} : (tensor<16x1x32x32xf32>) -> tensor<16x1x32x32xf32>
    %3 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "bcast_add_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "bcast_add_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q6 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 5.390495e+01 : f32, name = "data0_quant_i8"} : (tensor<16x256x32x32xf32>) -> tensor<16x256x32x32xsi8>
    %q7 = "tpu.quant"(%2) {from = "NONE", to = "INT8", scale = 0x422EE485 : f32, name = "data1_quant_i8"} : (tensor<16x1x32x32xf32>) -> tensor<16x1x32x32xsi8>
    %4 = "tpu.broadcast_add"(%q6, %q7, %3, %3, %q0, %q1) {name = "bcast_add", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 2.308060e+00 : f32}} : (tensor<16x256x32x32xsi8>, tensor<16x1x32x32xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<16x256x32x32xsi8>
    %q2 = "tpu.load_weight"(%0) {name = "bcast_sub_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q3 = "tpu.load_weight"(%0) {name = "bcast_sub_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %5 = "tpu.broadcast_sub"(%q6, %q7, %3, %3, %q2, %q3) {name = "bcast_sub", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 2.858630e+00 : f32}} : (tensor<16x256x32x32xsi8>, tensor<16x1x32x32xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<16x256x32x32xsi8>
    %q4 = "tpu.load_weight"(%0) {name = "bcast_mul_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q5 = "tpu.load_weight"(%0) {name = "bcast_mul_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %6 = "tpu.broadcast_mul"(%q6, %q7, %3, %3, %q4, %q5) {name = "bcast_mul", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 3.083220e+00 : f32}} : (tensor<16x256x32x32xsi8>, tensor<16x1x32x32xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<16x256x32x32xsi8>
    %q8 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 0x3C93B741 : f32, name = "bcast_add_dequant"} : (tensor<16x256x32x32xsi8>) -> tensor<16x256x32x32xf32>
    %q9 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3CB6F3CB : f32, name = "bcast_sub_dequant"} : (tensor<16x256x32x32xsi8>) -> tensor<16x256x32x32xf32>
    %q10 = "tpu.quant"(%6) {from = "INT8", to = "NONE", scale = 0x3CC5537A : f32, name = "bcast_mul_dequant"} : (tensor<16x256x32x32xsi8>) -> tensor<16x256x32x32xf32>
    return %q8, %q9, %q10 : tensor<16x256x32x32xf32>, tensor<16x256x32x32xf32>, tensor<16x256x32x32xf32>
  }
}
