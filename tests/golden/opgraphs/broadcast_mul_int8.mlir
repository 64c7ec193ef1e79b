module {
  func @tpu_func(%arg0: tensor<4x64x28x28xf32>, %arg1: tensor<4x64xf32>) -> tensor<4x64x28x28xf32> {
    %q0 = "tpu.weight_file"() {filename = "broadcast_mul_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data0", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.296740e+00 : f32}} : (tensor<4x64x28x28xf32>) -> tensor<4x64x28x28xf32>
    %2 = "tpu.input"(%arg1) {name = "data1", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 3.094830e+00 : f32}} : (tensor<4x64xf32>) -> tensor<4x64xf32>
    %3 = "tpu.none"() : () -> none
    %q1 = "tpu.load_weight"(%q0) {name = "bcast_mul_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.load_weight"(%q0) {name = "bcast_mul_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q3 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x421B4E10 : f32, name = "data0_quant_i8"} : (tensor<4x64x28x28xf32>) -> tensor<4x64x28x28xsi8>
    %q4 = "tpu.quant"(%2) {from = "NONE", to = "INT8", scale = 4.135930e+01 : f32, name = "data1_quant_i8"} : (tensor<4x64xf32>) -> tensor<4x64xsi8>
    %4 = "tpu.broadcast_mul"(%q3, %q4, %3, %3, %q1, %q2) {name = "bcast_mul", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 1.075710e+00 : f32}} : (tensor<4x64x28x28xsi8>, tensor<4x64xsi8>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<4x64x28x28xsi8>
    %q5 = "tpu.quant"(%4) {from = "INT8", to = "NONE", scale = 8.403985e-03 : f32, name = "bcast_mul_dequant"} : (tensor<4x64x28x28xsi8>) -> tensor<4x64x28x28xf32>
    return %q5 : tensor<4x64x28x28xf32>
  }
}
