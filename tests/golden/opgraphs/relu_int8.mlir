module {
  func @tpu_func(%arg0: tensor<32x16x224x224xf32>) -> (tensor<32x16x224x224xf32>, tensor<32x16x224x224xf32>, tensor<32x16x224x224xf32>) {
    %0 = "tpu.weight_file"() {filename = "relu_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.814910e+00 : f32}} : (tensor<32x16x224x224xf32>) -> tensor<32x16x224x224xf32>
    %2 = "tpu.none"() : () -> none
    %3 = "tpu.load_weight"(%0) {name = "slope_negative_slope", storage = "INT8"} : (memref<10xf32>) -> tensor<1x16x1x1xf32>
    %q7 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x420635D3 : f32, name = "data_quant_i8"} : (tensor<32x16x224x224xf32>) -> tensor<32x16x224x224xsi8>
    %4 = "tpu.relu"(%q7) {name = "relu", quant = {mode = "INT8", param_type = "NONE", threshold = 3.814910e+00 : f32}} : (tensor<32x16x224x224xsi8>) -> tensor<32x16x224x224xsi8>
    %q0 = "tpu.load_weight"(%0) {name = "leaky_relu_rshift_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "leaky_relu_multiplier_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.load_weight"(%0) {name = "leaky_relu_rshift_neg", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q3 = "tpu.load_weight"(%0) {name = "leaky_relu_multiplier_neg", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %5 = "tpu.leaky_relu"(%q7, %2, %2, %2, %2, %q0, %q1, %q2, %q3) {name = "leaky_relu", negative_slope = 1.000000e-01 : f32, quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.814910e+00 : f32}} : (tensor<32x16x224x224xsi8>, none, none, none, none, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>) -> tensor<32x16x224x224xsi8>
    %q4 = "tpu.load_weight"(%0) {name = "prelu_rshift_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q5 = "tpu.load_weight"(%0) {name = "prelu_multiplier_pos", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q6 = "tpu.load_weight"(%0) {name = "prelu_rshift_neg", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %6 = "tpu.prelu"(%q7, %3, %2, %2, %2, %2, %q4, %q5, %q6, %2) {name = "prelu", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I8", threshold = 3.253600e+00 : f32}} : (tensor<32x16x224x224xsi8>, tensor<1x16x1x1xf32>, none, none, none, none, tensor<1xf32>, tensor<1xf32>, tensor<1xf32>, none) -> tensor<32x16x224x224xsi8>
    %q8 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 0x3CF4277C : f32, name = "relu_dequant"} : (tensor<32x16x224x224xsi8>) -> tensor<32x16x224x224xf32>
    %q9 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3CF4277C : f32, name = "leaky_relu_dequant"} : (tensor<32x16x224x224xsi8>) -> tensor<32x16x224x224xf32>
    %q10 = "tpu.quant"(%6) {from = "INT8", to = "NONE", scale = 2.541875e-02 : f32, name = "prelu_dequant"} : (tensor<32x16x224x224xsi8>) -> tensor<32x16x224x224xf32>
    return %q8, %q9, %q10 : tensor<32x16x224x224xf32>, tensor<32x16x224x224xf32>, tensor<32x16x224x224xf32>
  }
}
