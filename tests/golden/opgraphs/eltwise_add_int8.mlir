module {
  func @tpu_func(%arg0: tensor<4x512x28x28xf32>, %arg1: tensor<4x512x28x28xf32>) -> tensor<4x512x28x28xf32> {
    %0 = "tpu.weight_file"() {filename = "eltwise_add_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data0", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.654240e+00 : f32}} : (tensor<4x512x28x28xf32>) -> tensor<4x512x28x28xf32>
    %2 = "tpu.input"(%arg1) {name = "data1", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.483370e+00 : f32}} : (tensor<4x512x28x28xf32>) -> tensor<4x512x28x28xf32>
    %3 = "tpu.none"() : () -> none
    %q0 = "tpu.load_weight"(%0) {name = "res3a_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "res3a_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<2xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x4240E61F : f32, name = "data0_quant_i8"} : (tensor<4x512x28x28xf32>) -> tensor<4x512x28x28xsi8>
    %q3 = "tpu.quant"(%2) {from = "NONE", to = "INT8", scale = 0x4212FBEE : f32, name = "data1_quant_i8"} : (tensor<4x512x28x28xf32>) -> tensor<4x512x28x28xsi8>
    %4 = "tpu.eltwise_add"(%q2, %q3, %3, %3, %q0, %q1) {name = "res3a", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.325260e+00 : f32}} : (tensor<4x512x28x28xsi8>, tensor<4x512x28x28xsi8>, none, none, tensor<1xf32>, tensor<2xf32>) -> tensor<4x512x28x28xsi8>
    %q4 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 0x3CD4D10F : f32, name = "res3a_dequant"} : (tensor<4x512x28x28xsi8>) -> tensor<4x512x28x28xf32>
    return %q4 : tensor<4x512x28x28xf32>
  }
}
