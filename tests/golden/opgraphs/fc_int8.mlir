module {
  func @tpu_func(%arg0: tensor<16x1x2048xf32>) -> tensor<16x1x400xf32> {
    %0 = "tpu.weight_file"() {filename = "fc_int8_weights.npz"} : () -> memref<10xf32>
    %1 = "tpu.input"(%arg0) {name = "data", quant = {mode = "NONE", param_type = "THRESHOLD", threshold = 2.461680e+00 : f32}} : (tensor<16x1x2048xf32>) -> tensor<16x1x2048xf32>
    %2 = "tpu.none"() : () -> none
    %3 = "tpu.load_weight"(%0) {name = "filter_quant", storage = "INT8"} : (memref<10xf32>) -> tensor<400x2048xf32>
    %4 = "tpu.load_weight"(%0) {name = "bias_quant", storage = "INT32"} : (memref<10xf32>) -> tensor<400xf32>
    %q0 = "tpu.load_weight"(%0) {name = "fc_rshift", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q1 = "tpu.load_weight"(%0) {name = "fc_multiplier", storage = "NONE"} : (memref<10xf32>) -> tensor<1xf32>
    %q2 = "tpu.quant"(%1) {from = "NONE", to = "INT8", scale = 0x424FFCF1 : f32, name = "data_quant_i8"} : (tensor<16x1x2048xf32>) -> tensor<16x1x2048xsi8>
    %5 = "tpu.fully_connected"(%q2, %3, %4, %2, %2, %q0, %q1) {name = "fc", quant = {mode = "INT8", param_type = "RSHIFT_AND_M_I32", threshold = 3.737270e+00 : f32}} : (tensor<16x1x2048xsi8>, tensor<400x2048xf32>, tensor<400xf32>, none, none, tensor<1xf32>, tensor<1xf32>) -> tensor<16x1x400xsi8>
    %q3 = "tpu.quant"(%5) {from = "INT8", to = "NONE", scale = 0x3CEF2F6F : f32, name = "fc_dequant"} : (tensor<16x1x400xsi8>) -> tensor<16x1x400xf32>
    return %q3 : tensor<16x1x400xf32>
  }
}
