module {
  func @tpu_func(%arg0: tensor<4x64x56x56xf32>) -> tensor<4x64x56x56xf32> {
    %0 = "tpu.weight_file"() {filename = "lrn_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.585790e+00 : f32}} : (tensor<4x64x56x56xf32>) -> tensor<4x64x56x56xf32>
    %2 = "tpu.none"() : () -> none
    %3 = "tpu.load_weight"(%0) {name = "slope_negative_slope", storage = "INT8"} : (memref<10xf32>) -> tensor<1x64x1x1xf32>
    %q0 = "tpu.load_weight"(%0) {name = "prelu_rshift_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "prelu_multiplier_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.load_weight"(%0) {name = "prelu_rshift_neg", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q5 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x42460159 : f32, name = "data_quant_i8"} : (tensor<4x64x56x56xf32>) -> tensor<4x64x56x56xsi8>
    %4 = "tpu.prelu"(%q5, %3, %2, %2, %2, %2, %q0, %q1, %q2, %2) {name = "prelu", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.314980e+00 : f32}} : (tensor<4x64x56x56xsi8>, tensor<1x64x1x1xf32>, none, none, none, none, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>, none) -> tensor<4x64x56x56xsi8>
    %5 = "tpu.relu"(%4) {name = "relu", quant = {mode = "INT8", param_type = "NONE", threshold = 3.314980e+00 : f32}} : (tensor<4x64x56x56xsi8>) -> tensor<4x64x56x56xsi8>
    %q3 = "tpu.load_weight"(%0) {name = "lrn_test_sq_gen_weight", storage = "UINT8"} : (memref<10xf32>) -> tensor<1x32x16x16xf32>
    %q4 = "tpu.load_weight"(%0) {name = "lrn_test_power_gen_weight", storage = "UINT8"} : (memref<10xf32>) -> tensor<1x32x16x16xf32>
    %9 = "tpu.lrn"(%5, %q3, %q4, %2) {alpha = 1.000000e-04 : f32, beta = 7.500000e-01 : f32, k = 1.000000e+00 : f32, local_size = 5 : i32, lrn_rshift = 14 : i32, name = "lrn_test", norm_region = 0 : i32, quant = {mode = "INT8", param_type = "THRESHOLD", threshold = 1.470710e+00 : f32}, quant_data0 = 205 : i32, quant_data1 = 144 : i32, sum_rshift = 10 : i32, threshold_parts = [0x3966755C : f32, 0x3A90095A : f32, 1.000000e+00 : f32]} : (tensor<4x64x56x56xsi8>, tensor<1x32x16x16xf32>, tensor<1x32x16x16xf32>, none) -> tensor<4x64x56x56xsi8>
    %q6 = "tpu.quant"(%9) {from = "INT8", to = "NONE", scale = 0x3C3C403A : f32, name = "lrn_test_dequant"} : (tensor<4x64x56x56xsi8>) -> tensor<4x64x56x56xf32>
    return %q6 : tensor<4x64x56x56xf32>
  }
}
